/*
 * qlin_api.hip - the C ABI of libqlinear (declared in include/qlinear.h).
 *
 * This layer owns the device, one stream, the weight registry and the staging buffers of the
 * host-pointer entry points, checks every argument the kernels rely on (whole blocks,
 * alignment, sizes) and turns HIP failures into status codes. It contains no arithmetic and
 * no CPU fallback: if the GPU cannot be used every call fails.
 */
#include "../../include/qlinear.h"
#include "../../include/qlinear_bench.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <atomic>
#include <map>
#include <vector>
#include <mutex>
#include <string>

#include "qlin_device.h"
#include "qlin_internal.h"

namespace {

using namespace qlin;

thread_local std::string t_error;

/* qlin_timer_begin / _end: the event pair belongs to the calling thread, so that threads timing their own streams do
 * not overwrite each other's start event; it goes when the thread ends or calls qlin_shutdown */
struct ThreadTimer {
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    bool begun = false;
    void reset() {
        if (ev0) (void)hipEventDestroy(ev0);
        if (ev1) (void)hipEventDestroy(ev1);
        ev0 = ev1 = nullptr;
        begun = false;
    }
    ~ThreadTimer() { reset(); }
};
thread_local ThreadTimer t_timer;

int fail(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    t_error = buf;
    return code;
}

}  // namespace

namespace qlin {
/* for the other translation units of the library: sets the text qlin_last_error() returns */
int set_error(int code, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    t_error = buf;
    return code;
}
}  // namespace qlin

namespace {

#define HIP_TRY(expr)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess)                                                                  \
            return fail(QLIN_ERR_DEVICE, "%s failed: %s", #expr, hipGetErrorString(e_));       \
    } while (0)

/* grow-only device buffer for staging */
struct DevBuf {
    void *p = nullptr;
    size_t cap = 0;
    int ensure(size_t n) {
        if (n <= cap) return QLIN_OK;
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
        size_t want = n + n / 4 + 256;
        if (hipMalloc(&p, want) != hipSuccess) {
            p = nullptr;
            return fail(QLIN_ERR_NOMEM, "hipMalloc of %zu bytes failed", want);
        }
        cap = want;
        return QLIN_OK;
    }
    void release() {
        if (p) (void)hipFree(p);
        p = nullptr;
        cap = 0;
    }
};

struct Range { size_t bytes; void *dev; };
constexpr size_t kPinnedHalf = (size_t)2 << 20; /* bytes of pinned staging per direction */

struct State {
    std::mutex mu;
    bool ready = false;
    int device = 0;
    int n_cu = 256;
    hipStream_t stream = nullptr;
    std::map<uintptr_t, Range> registry; /* host begin -> range */
    DevBuf w[3], x, y[3], tmp[4];
    /* pinned host staging for the small per-call transfers of the host-pointer entry points (x up, y down):
     * a copy between pageable memory and the GPU is staged and waited for by the runtime one at a time */
    uint8_t *pinned = nullptr;
    uint8_t *pinned_dev = nullptr; /* the same buffer as kernels address it; null: results come by the runtime's copy */
    size_t up_used = 0, down_used = 0;
    struct Pending { void *host; const void *staged; size_t bytes; };
    std::vector<Pending> pending;
    /* 0: the vendor library, 1: this library's tile kernel, 2: neither (the vector-ALU kernel); read by device-pointer
     * calls outside the lock */
    std::atomic<int> dense_gemm_mode{0}; /* bf16 products by the vendor library (faster) unless QLIN_DENSE_GEMM=own or
                                            qlin_set_dense_gemm_own say otherwise */
    bool prefill_bf16 = false; /* qlin_gemm_tokenmajor on the matrix cores (opt-in: costs accuracy) */
} g;

int ensure_init_locked(int device) {
    if (!g.pending.empty() || g.up_used || g.down_used) { /* left by a call that failed before it finished */
        /* its kernels may still be reading or writing the staging regions that the offsets are about to hand out again */
        if (g.stream) (void)hipStreamSynchronize(g.stream);
        g.pending.clear();
        g.up_used = g.down_used = 0;
    }
    if (g.ready) return QLIN_OK;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0)
        return fail(QLIN_ERR_DEVICE, "no HIP device available (this library has no CPU path)");
    if (device < 0 || device >= count) return fail(QLIN_ERR_ARG, "device %d out of range (%d devices)", device, count);
    HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, device));
    g.n_cu = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    HIP_TRY(hipStreamCreate(&g.stream));
    g.device = device;
    if (const char *e = getenv("QLIN_PREFILL_MATRIX_CORES")) g.prefill_bf16 = e[0] == '1';
    if (const char *e = getenv("QLIN_DENSE_GEMM")) g.dense_gemm_mode = e[0] == 'o' ? 1 : 0;
    if (hipHostMalloc((void **)&g.pinned, 2 * kPinnedHalf, hipHostMallocMapped) != hipSuccess) {
        g.pinned = nullptr; /* transfers then go straight from and to the caller's memory */
        (void)hipGetLastError();
    } else if (hipHostGetDevicePointer((void **)&g.pinned_dev, g.pinned, 0) != hipSuccess) {
        g.pinned_dev = nullptr;
        (void)hipGetLastError();
    }
    /* address of the no-allocation entry point's scratch on this device */
    if (hipError_t e = moe_static_scratch_setup(device); e != hipSuccess) {
        /* a retry starts from nothing: no second stream, no second staging buffer */
        if (g.pinned) (void)hipHostFree(g.pinned);
        g.pinned = g.pinned_dev = nullptr;
        (void)hipStreamDestroy(g.stream);
        g.stream = nullptr;
        return fail(QLIN_ERR_DEVICE, "looking up the built-in scratch failed: %s", hipGetErrorString(e));
    }
    g.ready = true;
    return QLIN_OK;
}

bool known_type(uint32_t t) {
    int be, bb;
    return type_geometry(t, &be, &bb);
}
bool block_type(uint32_t t) {
    int be, bb;
    return type_geometry(t, &be, &bb) && be > 1;
}
size_t row_size(uint32_t t, int n) {
    int be, bb;
    if (!type_geometry(t, &be, &bb) || n < 0) return 0;
    return (size_t)((n + be - 1) / be) * (size_t)bb;
}
bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

/* device pointer mirroring a host pointer inside a registered range, or nullptr */
const void *lookup_locked(const void *host, size_t need) {
    if (g.registry.empty()) return nullptr;
    const uintptr_t h = reinterpret_cast<uintptr_t>(host);
    auto it = g.registry.upper_bound(h);
    if (it == g.registry.begin()) return nullptr;
    --it;
    if (h < it->first || h + need > it->first + it->second.bytes) return nullptr;
    return static_cast<const uint8_t *>(it->second.dev) + (h - it->first);
}

/* host -> device on the library's stream; small transfers go through the pinned buffer */
/* Results go to the pinned buffer by a kernel that stores over the bus, not by the runtime's device-to-host
 * copy: after a process has freed a few GiB of device memory that copy took 95 us instead of 9.5 us for the
 * 57 KB of a matvec result (until another stream was created), which made a 35 us call a 130 us call. */
__global__ void __launch_bounds__(256) copy16_kernel(uint8_t *__restrict__ dst, const uint8_t *__restrict__ src,
                                                            size_t bytes) {
    const size_t n16 = bytes >> 4;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256)
        reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(src)[i];
    if (blockIdx.x == 0 && threadIdx.x < (bytes & 15)) dst[(n16 << 4) + threadIdx.x] = src[(n16 << 4) + threadIdx.x];
}

int upload_locked(void *dev, const void *host, size_t bytes) {
    const size_t need = (bytes + 255) & ~(size_t)255;
    if (g.pinned && g.up_used + need <= kPinnedHalf) {
        uint8_t *st = g.pinned + g.up_used;
        g.up_used += need;
        memcpy(st, host, bytes);
        if (g.pinned_dev && aligned(dev, 16) && bytes <= (1u << 20)) {
            /* small inputs (an activation vector): a kernel that reads the staging buffer over the bus, for the
             * reason given at copy16_kernel and because it starts sooner than the runtime's copy */
            const size_t groups = ((bytes >> 4) + 255) / 256;
            const int grid = (int)std::min<size_t>(std::max<size_t>(groups, 1), 64);
            copy16_kernel<<<grid, 256, 0, g.stream>>>(static_cast<uint8_t *>(dev), g.pinned_dev + (st - g.pinned), bytes);
            HIP_TRY(hipGetLastError());
        } else {
            HIP_TRY(hipMemcpyAsync(dev, st, bytes, hipMemcpyHostToDevice, g.stream));
        }
    } else {
        HIP_TRY(hipMemcpyAsync(dev, host, bytes, hipMemcpyHostToDevice, g.stream));
    }
    return QLIN_OK;
}
/* device -> host on the library's stream; the bytes are in `host` after finish_locked() */
int download_locked(void *host, const void *dev, size_t bytes) {
    const size_t need = (bytes + 255) & ~(size_t)255;
    if (bytes == 0) return QLIN_OK;
    if (g.pinned && g.down_used + need <= kPinnedHalf) {
        uint8_t *st = g.pinned + kPinnedHalf + g.down_used;
        g.down_used += need;
        if (g.pinned_dev && aligned(dev, 16)) {
            const size_t groups = ((bytes >> 4) + 255) / 256;
            const int grid = (int)std::min<size_t>(std::max<size_t>(groups, 1), 64);
            copy16_kernel<<<grid, 256, 0, g.stream>>>(g.pinned_dev + (st - g.pinned),
                                                             static_cast<const uint8_t *>(dev), bytes);
            HIP_TRY(hipGetLastError());
        } else {
            HIP_TRY(hipMemcpyAsync(st, dev, bytes, hipMemcpyDeviceToHost, g.stream));
        }
        g.pending.push_back({host, st, bytes});
    } else {
        HIP_TRY(hipMemcpyAsync(host, dev, bytes, hipMemcpyDeviceToHost, g.stream));
    }
    return QLIN_OK;
}
/* waits for the library's stream and hands the staged results over */
int finish_locked() {
    const hipError_t e = hipStreamSynchronize(g.stream);
    if (e == hipSuccess)
        for (const State::Pending &pd : g.pending) memcpy(pd.host, pd.staged, pd.bytes);
    g.pending.clear();
    g.up_used = g.down_used = 0;
    if (e != hipSuccess) return fail(QLIN_ERR_DEVICE, "hipStreamSynchronize failed: %s", hipGetErrorString(e));
    return QLIN_OK;
}

/* device view of host weights: the registered copy, or a staged copy in `buf` */
int weights_on_device_locked(const void *host, size_t bytes, DevBuf &buf, const void **dev) {
    if (const void *d = lookup_locked(host, bytes)) {
        *dev = d;
        return QLIN_OK;
    }
    if (int rc = buf.ensure(bytes)) return rc;
    HIP_TRY(hipMemcpyAsync(buf.p, host, bytes, hipMemcpyHostToDevice, g.stream));
    *dev = buf.p;
    return QLIN_OK;
}

/* the tuned kernels, on packed rows (row_stride 0) or on a column range of longer rows; false: none takes the shape */
static bool launch_gemv_tuned(uint32_t type, const GemvJob &job, const float *x, int n_cols, size_t row_stride,
                              hipStream_t s, hipError_t *err) {
    bool w_aligned = true;
    for (int m = 0; m < job.n_mat; m++) w_aligned = w_aligned && aligned(job.W[m], 16);
    if (type == T_Q4_K && n_cols % 256 == 0 && n_cols <= 16384 && w_aligned && aligned(x, 16)) {
        *err = launch_gemv_q4k(job, x, n_cols, s, g.n_cu, row_stride);
        return true;
    }
    if (launch_gemv_dense_long(type, job, x, n_cols, g.n_cu, s, err, row_stride)) return true;
    if (launch_gemv_grid(type, job, x, n_cols, g.n_cu, s, err, row_stride)) return true;
    if (launch_gemv_int(type, job, x, n_cols, g.n_cu, s, err, row_stride)) return true;
    return launch_gemv_stream(type, job, x, n_cols, g.n_cu, s, err, row_stride);
}

/* Rows too long for the tuned kernels (more than 16384 elements or 8 KB) as column ranges of at most `cap`
 * elements, each a launch of its own over the full rows' pitch: the first with the job's mode, the others adding
 * to y in stream order. 0: the type or the shape does not split that way. */
static int column_range(uint32_t type, int n_cols) {
    int be, bb;
    type_geometry(type, &be, &bb);
    /* a range is whole 256-element groups; for the kernels that want rows on 16-byte boundaries also so many
     * blocks that their bytes are a multiple of 16 */
    const bool any_address = gemv_int_takes_any_even_address(type);
    int granule = be;
    while (granule % 256 != 0 || (!any_address && ((size_t)(granule / be) * bb) % 16 != 0)) granule += be;
    if (n_cols % granule != 0) return 0;
    /* Q4_K: what its kernel takes; the others: the longest range whose x stays in the lanes' registers */
    const bool dense = type == T_F32 || type == T_F16 || type == T_BF16;
    const int cap = (type == T_Q4_K || gemv_grid_covers(type) || dense) ? 16384 : 4096; /* the long-row kernels' limit */
    int range = cap / granule * granule;
    while (cap == 4096 && range > 0 && (size_t)(range / be) * bb > 8192) range -= granule; /* those kernels' row images */
    if (range <= 0) return 0;
    const int n_ranges = (n_cols + range - 1) / range;
    range = ((n_cols + n_ranges - 1) / n_ranges + granule - 1) / granule * granule; /* ranges of about equal length */
    return range;
}

/* shape-based choice: tuned Q4_K kernel, else the matrix-instruction kernel for long rows of the codebook formats,
 * else the integer-dot kernel (formats with small integer codes), else the streaming float kernel, else - rows
 * too long for those - the same kernels over column ranges, else (ragged shapes, unaligned pointers) the plain kernel */
hipError_t dispatch_gemv_job(uint32_t type, const GemvJob &job, const float *x, int n_cols, hipStream_t s) {
    if ((job.mode == kSiluMul ? job.n_rows[0] : job.total_rows()) == 0) return hipSuccess;
    bool w_aligned = true;
    for (int m = 0; m < job.n_mat; m++) w_aligned = w_aligned && aligned(job.W[m], 16);
    if ((type == T_F16 || type == T_BF16 || type == T_F32) && (n_cols % 8 != 0 || !w_aligned))
        return launch_gemv_dense_ragged(type, job, x, n_cols, s); /* rows that are not whole 16-byte groups */
    hipError_t err;
    if (launch_gemv_tuned(type, job, x, n_cols, 0, s, &err)) return err;
    int be, bb;
    type_geometry(type, &be, &bb);
    const size_t row_bytes = (size_t)(n_cols / be) * bb;
    const int range = (job.mode != kSiluMul && w_aligned && aligned(x, 16) && n_cols % be == 0 &&
                       (row_bytes % 16 == 0 || gemv_int_takes_any_even_address(type)))
                          ? column_range(type, n_cols) : 0;
    if (range > 0 && range < n_cols) {
        for (int c0 = 0; c0 < n_cols; c0 += range) {
            GemvJob part = job;
            for (int m = 0; m < job.n_mat; m++) part.W[m] = (const uint8_t *)job.W[m] + (size_t)(c0 / be) * bb;
            if (c0 > 0) part.mode = kAdd;
            const int cols = n_cols - c0 < range ? n_cols - c0 : range;
            if (!launch_gemv_tuned(type, part, x + c0, cols, row_bytes, s, &err)) {
                /* every range has the shape of the first or is shorter: cannot happen once the first was taken */
                if (c0 == 0) return launch_gemv_generic(type, job, x, n_cols, s);
                return hipErrorInvalidValue;
            }
            if (err != hipSuccess) return err;
        }
        return hipSuccess;
    }
    return launch_gemv_generic(type, job, x, n_cols, s);
}
hipError_t dispatch_gemv(uint32_t type, const void *W, const float *x, float *y, int n_rows,
                         int n_cols, hipStream_t s) {
    return dispatch_gemv_job(type, single_job(W, y, n_rows), x, n_cols, s);
}

/* any_dense_length: the matvec paths take dense F32/F16/BF16 rows of any length, as tf_qmatvec does
 * (common/transformer.h:1049-1114); the GEMM and MoE paths want whole groups of eight elements */
int check_linear_shape(uint32_t type, int n_rows, int n_cols, bool any_dense_length = false) {
    int be, bb;
    if (!type_geometry(type, &be, &bb))
        return fail(QLIN_ERR_TYPE, "unsupported weight type %u", type);
    if (be == 1 && !any_dense_length) be = 8; /* dense rows go through those kernels eight elements at a time */
    if (n_rows < 0 || n_cols <= 0) return fail(QLIN_ERR_ARG, "bad shape %d x %d", n_rows, n_cols);
    if (n_cols % be) return fail(QLIN_ERR_ARG, "n_cols %d is not a whole number of %d-element blocks", n_cols, be);
    return QLIN_OK;
}

int matvec_host_locked(float *dst, const void *W, uint32_t type, int n_cols, const float *x, int n_rows,
                       int slot, bool upload_x) {
    const size_t rb = row_size(type, n_cols);
    const void *dW;
    if (int rc = weights_on_device_locked(W, rb * (size_t)n_rows, g.w[slot], &dW)) return rc;
    if (upload_x) {
        if (int rc = g.x.ensure((size_t)n_cols * 4)) return rc;
        if (int rc = upload_locked(g.x.p, x, (size_t)n_cols * 4)) return rc;
    }
    /* the tuned Q4_K kernel stores a workgroup's results as one run of consecutive floats: it can write them
     * straight into the pinned result buffer over the bus, which saves the copy kernel behind it */
    const size_t y_bytes = (size_t)n_rows * 4, y_need = (y_bytes + 255) & ~(size_t)255;
    if (type == T_Q4_K && n_cols % 256 == 0 && n_cols <= 16384 && aligned(dW, 16) && g.pinned_dev &&
        g.down_used + y_need <= kPinnedHalf) {
        uint8_t *st = g.pinned + kPinnedHalf + g.down_used;
        g.down_used += y_need;
        HIP_TRY(dispatch_gemv(type, dW, (const float *)g.x.p, (float *)(g.pinned_dev + (st - g.pinned)), n_rows, n_cols, g.stream));
        g.pending.push_back({dst, st, y_bytes});
        return QLIN_OK;
    }
    if (int rc = g.y[slot].ensure(y_bytes + 16)) return rc;
    HIP_TRY(dispatch_gemv(type, dW, (const float *)g.x.p, (float *)g.y[slot].p, n_rows, n_cols, g.stream));
    if (int rc = download_locked(dst, g.y[slot].p, y_bytes)) return rc;
    return QLIN_OK;
}

/* up to three matrices against one x (host pointers). Matrices of one type go out as ONE launch;
 * otherwise one launch per matrix, with the SiLU product as a separate pass. dst[m] receives
 * n_rows[m] floats (mode kSiluMul: dst[0] only; mode kAdd: dst[m] is read first). */
int matvec_multi_host_locked(int n_mat, float *const dst[3], const void *const W[3], const uint32_t types[3],
                             const int n_rows[3], int n_cols, const float *x, int mode) {
    if (int rc = g.x.ensure((size_t)n_cols * 4)) return rc;
    if (int rc = upload_locked(g.x.p, x, (size_t)n_cols * 4)) return rc;
    const void *dW[3] = {nullptr, nullptr, nullptr};
    bool same = true;
    for (int m = 0; m < n_mat; m++) {
        if (n_rows[m] == 0) continue;
        if (int rc = weights_on_device_locked(W[m], row_size(types[m], n_cols) * (size_t)n_rows[m], g.w[m], &dW[m])) return rc;
        if (int rc = g.y[m].ensure((size_t)n_rows[m] * 4 + 16)) return rc;
        same = same && types[m] == types[0];
    }
    if (mode == kAdd)
        for (int m = 0; m < n_mat; m++)
            if (n_rows[m]) { if (int rc = upload_locked(g.y[m].p, dst[m], (size_t)n_rows[m] * 4)) return rc; }
    const float *dx = (const float *)g.x.p;
    if (same && n_rows[0] > 0) {
        GemvJob job = {{dW[0], dW[1], dW[2]}, {(float *)g.y[0].p, (float *)g.y[1].p, (float *)g.y[2].p},
                       {n_rows[0], n_rows[1], n_rows[2]}, n_mat, mode};
        HIP_TRY(dispatch_gemv_job(types[0], job, dx, n_cols, g.stream));
    } else {
        for (int m = 0; m < n_mat; m++)
            if (n_rows[m])
                HIP_TRY(dispatch_gemv_job(types[m], single_job(dW[m], (float *)g.y[m].p, n_rows[m], mode == kAdd ? kAdd : kStore),
                                          dx, n_cols, g.stream));
        if (mode == kSiluMul)
            HIP_TRY(launch_silu_mul((float *)g.y[0].p, (const float *)g.y[0].p, (const float *)g.y[1].p, n_rows[0], g.stream));
    }
    const int n_out = mode == kSiluMul ? 1 : n_mat;
    for (int m = 0; m < n_out; m++)
        if (n_rows[m]) { if (int rc = download_locked(dst[m], g.y[m].p, (size_t)n_rows[m] * 4)) return rc; }
    return QLIN_OK;
}

bool dense_type(uint32_t t) { return t == T_F16 || t == T_BF16 || t == T_F32; }

/* argument checks shared by the device-resident matvec entry points */
int check_dev_gemv(uint32_t type, int n_rows, int n_cols, const void *W, const float *x, const float *y) {
    if (int rc = check_linear_shape(type, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!W || !x || !y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, type == T_F32 ? 4 : 2) || !aligned(x, 16) || !aligned(y, 4))
        return fail(QLIN_ERR_ARG, "W needs 2-byte (F32: 4-byte), x 16-byte, y 4-byte alignment");
    return QLIN_OK;
}
int init_once() {
    std::lock_guard<std::mutex> lk(g.mu);
    return ensure_init_locked(0);
}

void void_decoder(uint32_t type, const char *name, const void *src, float *dst, int n) {
    const int rc = qlin_dequant_row(type, src, dst, n);
    if (rc != QLIN_OK) {
        fprintf(stderr, "%s: %s\n", name, qlin_last_error());
        if (dst && n > 0) memset(dst, 0, (size_t)n * sizeof(float));
    }
}

}  // namespace

extern "C" {

/* ------------------------------------------------------------------ lifecycle */

int qlin_init(int device) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (g.ready && device != g.device) return fail(QLIN_ERR_ARG, "already initialised on device %d", g.device);
    return ensure_init_locked(device);
}

void qlin_shutdown(void) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (!g.ready) return;
    (void)hipStreamSynchronize(g.stream);
    for (auto &kv : g.registry) (void)hipFree(kv.second.dev);
    g.registry.clear();
    for (auto &b : g.w) b.release();
    for (auto &b : g.y) b.release();
    for (auto &b : g.tmp) b.release();
    g.x.release();
    if (g.pinned) (void)hipHostFree(g.pinned);
    g.pinned = nullptr;
    g.pinned_dev = nullptr;
    g.pending.clear();
    g.up_used = g.down_used = 0;
    (void)hipStreamDestroy(g.stream);
    g.stream = nullptr;
    g.ready = false;
    t_timer.reset();
}

const char *qlin_last_error(void) { return t_error.c_str(); }

int qlin_device_info(char *name, size_t cap, int *compute_units, size_t *mem_bytes) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    hipDeviceProp_t prop;
    HIP_TRY(hipGetDeviceProperties(&prop, g.device));
    if (name && cap) {
        snprintf(name, cap, "%s (%s)", prop.name, prop.gcnArchName);
    }
    if (compute_units) *compute_units = prop.multiProcessorCount;
    if (mem_bytes) *mem_bytes = prop.totalGlobalMem;
    return QLIN_OK;
}

/* ------------------------------------------------------------------ codec */

size_t qlin_dequant_row_size(uint32_t ggml_type, int n) { return row_size(ggml_type, n); }

int qlin_dequant_rows(uint32_t ggml_type, const void *src, float *dst, int n_rows, int n_cols) {
    if (!known_type(ggml_type)) return fail(QLIN_ERR_TYPE, "unsupported type %u", ggml_type);
    if (n_rows < 0 || n_cols < 0) return fail(QLIN_ERR_ARG, "negative size");
    int be, bb;
    type_geometry(ggml_type, &be, &bb);
    const int whole = n_cols / be * be; /* a ragged tail is not decoded */
    if (n_rows == 0 || whole == 0) return QLIN_OK;
    if (!src || !dst) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const size_t rb = row_size(ggml_type, n_cols);
    const void *dW;
    if (int rc = weights_on_device_locked(src, rb * (size_t)(n_rows - 1) + (size_t)(whole / be) * bb, g.w[0], &dW)) return rc;
    const size_t out_bytes = (size_t)n_rows * n_cols * 4;
    if (int rc = g.tmp[0].ensure(out_bytes)) return rc;
    HIP_TRY(launch_dequant(ggml_type, dW, nullptr, 0, (float *)g.tmp[0].p, n_rows, n_cols, rb, g.stream));
    if (whole == n_cols) {
        HIP_TRY(hipMemcpyAsync(dst, g.tmp[0].p, out_bytes, hipMemcpyDeviceToHost, g.stream));
    } else { /* leave the undecoded tail of every row untouched in dst */
        HIP_TRY(hipMemcpy2DAsync(dst, (size_t)n_cols * 4, g.tmp[0].p, (size_t)n_cols * 4, (size_t)whole * 4,
                                 (size_t)n_rows, hipMemcpyDeviceToHost, g.stream));
    }
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_dequant_row(uint32_t ggml_type, const void *src, float *dst, int n) {
    return qlin_dequant_rows(ggml_type, src, dst, 1, n);
}

void qlin_dequantize_row_q8_0(const void *s, float *d, int n) { void_decoder(T_Q8_0, "qlin_dequantize_row_q8_0", s, d, n); }
void qlin_dequantize_row_q4_K(const void *s, float *d, int n) { void_decoder(T_Q4_K, "qlin_dequantize_row_q4_K", s, d, n); }
void qlin_dequantize_row_q5_K(const void *s, float *d, int n) { void_decoder(T_Q5_K, "qlin_dequantize_row_q5_K", s, d, n); }
void qlin_dequantize_row_q6_K(const void *s, float *d, int n) { void_decoder(T_Q6_K, "qlin_dequantize_row_q6_K", s, d, n); }
void qlin_dequantize_row_iq2_xxs(const void *s, float *d, int n) { void_decoder(T_IQ2_XXS, "qlin_dequantize_row_iq2_xxs", s, d, n); }
void qlin_dequantize_row_iq3_s(const void *s, float *d, int n) { void_decoder(T_IQ3_S, "qlin_dequantize_row_iq3_s", s, d, n); }
void qlin_dequantize_row_iq4_nl(const void *s, float *d, int n) { void_decoder(T_IQ4_NL, "qlin_dequantize_row_iq4_nl", s, d, n); }
void qlin_dequantize_row_q4_0(const void *s, float *d, int n) { void_decoder(T_Q4_0, "qlin_dequantize_row_q4_0", s, d, n); }
void qlin_dequantize_row_q4_1(const void *s, float *d, int n) { void_decoder(T_Q4_1, "qlin_dequantize_row_q4_1", s, d, n); }
void qlin_dequantize_row_q5_0(const void *s, float *d, int n) { void_decoder(T_Q5_0, "qlin_dequantize_row_q5_0", s, d, n); }
void qlin_dequantize_row_q5_1(const void *s, float *d, int n) { void_decoder(T_Q5_1, "qlin_dequantize_row_q5_1", s, d, n); }
void qlin_dequantize_row_q2_K(const void *s, float *d, int n) { void_decoder(T_Q2_K, "qlin_dequantize_row_q2_K", s, d, n); }
void qlin_dequantize_row_q3_K(const void *s, float *d, int n) { void_decoder(T_Q3_K, "qlin_dequantize_row_q3_K", s, d, n); }
void qlin_dequantize_row_q1_0(const void *s, float *d, int n) { void_decoder(T_Q1_0, "qlin_dequantize_row_q1_0", s, d, n); }
void qlin_dequantize_row_mxfp4(const void *s, float *d, int n) { void_decoder(T_MXFP4, "qlin_dequantize_row_mxfp4", s, d, n); }
void qlin_dequantize_row_nvfp4(const void *s, float *d, int n) { void_decoder(T_NVFP4, "qlin_dequantize_row_nvfp4", s, d, n); }
void qlin_dequantize_row_iq2_xs(const void *s, float *d, int n) { void_decoder(T_IQ2_XS, "qlin_dequantize_row_iq2_xs", s, d, n); }
void qlin_dequantize_row_iq2_s(const void *s, float *d, int n) { void_decoder(T_IQ2_S, "qlin_dequantize_row_iq2_s", s, d, n); }
void qlin_dequantize_row_iq3_xxs(const void *s, float *d, int n) { void_decoder(T_IQ3_XXS, "qlin_dequantize_row_iq3_xxs", s, d, n); }
void qlin_dequantize_row_iq4_xs(const void *s, float *d, int n) { void_decoder(T_IQ4_XS, "qlin_dequantize_row_iq4_xs", s, d, n); }
void qlin_dequantize_row_iq1_s(const void *s, float *d, int n) { void_decoder(T_IQ1_S, "qlin_dequantize_row_iq1_s", s, d, n); }
void qlin_dequantize_row_iq1_m(const void *s, float *d, int n) { void_decoder(T_IQ1_M, "qlin_dequantize_row_iq1_m", s, d, n); }
void qlin_dequantize_row_tq1_0(const void *s, float *d, int n) { void_decoder(T_TQ1_0, "qlin_dequantize_row_tq1_0", s, d, n); }
void qlin_dequantize_row_tq2_0(const void *s, float *d, int n) { void_decoder(T_TQ2_0, "qlin_dequantize_row_tq2_0", s, d, n); }
void qlin_dequantize_row_bf16(const void *s, float *d, int n) { void_decoder(T_BF16, "qlin_dequantize_row_bf16", s, d, n); }

/* ------------------------------------------------------------------ weights */

int qlin_weight_register(const void *host_data, size_t n_bytes) {
    if (!host_data || n_bytes == 0) return fail(QLIN_ERR_ARG, "null or empty weight range");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const uintptr_t h = reinterpret_cast<uintptr_t>(host_data);
    if (lookup_locked(host_data, 1) || lookup_locked((const uint8_t *)host_data + n_bytes - 1, 1))
        return fail(QLIN_ERR_ARG, "range overlaps a registered range");
    auto nxt = g.registry.lower_bound(h);
    if (nxt != g.registry.end() && nxt->first < h + n_bytes) return fail(QLIN_ERR_ARG, "range overlaps a registered range");
    void *dev = nullptr;
    if (hipMalloc(&dev, n_bytes + 256) != hipSuccess) return fail(QLIN_ERR_NOMEM, "hipMalloc of %zu bytes failed", n_bytes);
    hipError_t e = hipMemcpy(dev, host_data, n_bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail(QLIN_ERR_DEVICE, "upload failed: %s", hipGetErrorString(e));
    }
    g.registry[h] = Range{n_bytes, dev};
    return QLIN_OK;
}

int qlin_weight_adopt(const void *host_data, size_t n_bytes, void *dev_copy) {
    if (!host_data || n_bytes == 0 || !dev_copy) return fail(QLIN_ERR_ARG, "null or empty weight range");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const uintptr_t h = reinterpret_cast<uintptr_t>(host_data);
    if (lookup_locked(host_data, 1) || lookup_locked((const uint8_t *)host_data + n_bytes - 1, 1))
        return fail(QLIN_ERR_ARG, "range overlaps a registered range");
    auto nxt = g.registry.lower_bound(h);
    if (nxt != g.registry.end() && nxt->first < h + n_bytes) return fail(QLIN_ERR_ARG, "range overlaps a registered range");
    g.registry[h] = Range{n_bytes, dev_copy};
    return QLIN_OK;
}

int qlin_weight_unregister(const void *host_data) {
    std::lock_guard<std::mutex> lk(g.mu);
    auto it = g.registry.find(reinterpret_cast<uintptr_t>(host_data));
    if (it == g.registry.end()) return fail(QLIN_ERR_ARG, "pointer was not registered");
    if (g.ready) (void)hipStreamSynchronize(g.stream);
    (void)hipFree(it->second.dev);
    g.registry.erase(it);
    return QLIN_OK;
}

const void *qlin_weight_device_ptr(const void *host_ptr) {
    std::lock_guard<std::mutex> lk(g.mu);
    return lookup_locked(host_ptr, 1);
}

/* ------------------------------------------------------------------ linear, host pointers */

int qlin_matvec(float *dst, const void *W, uint32_t type, int n_cols, const float *x, int n_rows) {
    if (int rc = check_linear_shape(type, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!dst || !W || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    if (int rc = matvec_host_locked(dst, W, type, n_cols, x, n_rows, 0, true)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_matvec_fused2(float *dst1, const void *W1, uint32_t type1, float *dst2, const void *W2,
                       uint32_t type2, int n_cols, const float *x, int n_rows) {
    if (int rc = check_linear_shape(type1, n_rows, n_cols, true)) return rc;
    if (int rc = check_linear_shape(type2, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!dst1 || !dst2 || !W1 || !W2 || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const void *W[3] = {W1, W2, nullptr};
    const uint32_t types[3] = {type1, type2, 0};
    float *dst[3] = {dst1, dst2, nullptr};
    const int rows[3] = {n_rows, n_rows, 0};
    if (int rc = matvec_multi_host_locked(2, dst, W, types, rows, n_cols, x, kStore)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_matvec_qkv(float *q, const void *Wq, uint32_t type_q, int n_q, float *k, const void *Wk,
                    uint32_t type_k, float *v, const void *Wv, uint32_t type_v, int n_kv,
                    int n_cols, const float *x) {
    if (int rc = check_linear_shape(type_q, n_q, n_cols, true)) return rc;
    if (int rc = check_linear_shape(type_k, n_kv, n_cols, true)) return rc;
    if (int rc = check_linear_shape(type_v, n_kv, n_cols, true)) return rc;
    if (!x || (n_q && (!q || !Wq)) || (n_kv && (!k || !Wk || !v || !Wv))) return fail(QLIN_ERR_ARG, "null pointer");
    if (n_q == 0 && n_kv == 0) return QLIN_OK;
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const void *W[3] = {Wq, Wk, Wv};
    const uint32_t types[3] = {type_q, type_k, type_v};
    float *dst[3] = {q, k, v};
    const int rows[3] = {n_q, n_kv, n_kv};
    if (int rc = matvec_multi_host_locked(3, dst, W, types, rows, n_cols, x, kStore)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_matvec_silu_mul(float *dst, const void *Wgate, uint32_t type_gate, const void *Wup, uint32_t type_up,
                         int n_cols, const float *x, int n_rows) {
    if (int rc = check_linear_shape(type_gate, n_rows, n_cols, true)) return rc;
    if (int rc = check_linear_shape(type_up, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!dst || !Wgate || !Wup || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const void *W[3] = {Wgate, Wup, nullptr};
    const uint32_t types[3] = {type_gate, type_up, 0};
    float *out[3] = {dst, nullptr, nullptr};
    const int rows[3] = {n_rows, n_rows, 0};
    if (int rc = matvec_multi_host_locked(2, out, W, types, rows, n_cols, x, kSiluMul)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_matvec_add(float *dst, const void *W, uint32_t type, int n_cols, const float *x, int n_rows) {
    if (int rc = check_linear_shape(type, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!dst || !W || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const void *Wm[3] = {W, nullptr, nullptr};
    const uint32_t types[3] = {type, 0, 0};
    float *out[3] = {dst, nullptr, nullptr};
    const int rows[3] = {n_rows, 0, 0};
    if (int rc = matvec_multi_host_locked(1, out, Wm, types, rows, n_cols, x, kAdd)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_matvec_argmax(int *index, float *value, float *logits, const void *W, uint32_t type, int n_cols,
                       const float *x, int n_rows) {
    if (int rc = check_linear_shape(type, n_rows, n_cols, true)) return rc;
    if (n_rows == 0) return fail(QLIN_ERR_ARG, "argmax over no rows");
    if (!index || !W || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const size_t rb = row_size(type, n_cols);
    const void *dW;
    if (int rc = weights_on_device_locked(W, rb * (size_t)n_rows, g.w[0], &dW)) return rc;
    if (int rc = g.x.ensure((size_t)n_cols * 4)) return rc;
    if (int rc = upload_locked(g.x.p, x, (size_t)n_cols * 4)) return rc;
    if (int rc = g.y[0].ensure((size_t)n_rows * 4 + 16)) return rc;
    if (int rc = g.tmp[0].ensure(QLIN_ARGMAX_RESULT_BYTES)) return rc;
    HIP_TRY(dispatch_gemv(type, dW, (const float *)g.x.p, (float *)g.y[0].p, n_rows, n_cols, g.stream));
    HIP_TRY(launch_argmax((const float *)g.y[0].p, n_rows, (float *)g.tmp[0].p, g.stream));
    float res[2];
    if (int rc = download_locked(res, g.tmp[0].p, 8)) return rc;
    if (logits) { if (int rc = download_locked(logits, g.y[0].p, (size_t)n_rows * 4)) return rc; }
    if (int rc = finish_locked()) return rc;
    memcpy(index, &res[0], 4);
    if (value) *value = res[1];
    return QLIN_OK;
}

int qlin_matvec_expert(float *dst, const void *W, uint32_t type, int n_cols, int expert, const float *x,
                       int rows_per_expert) {
    if (int rc = check_linear_shape(type, rows_per_expert, n_cols, true)) return rc;
    if (expert < 0) return fail(QLIN_ERR_ARG, "negative expert index");
    if (!W) return fail(QLIN_ERR_ARG, "null pointer");
    const size_t rb = row_size(type, n_cols);
    const uint8_t *slice = (const uint8_t *)W + (size_t)expert * (size_t)rows_per_expert * rb;
    return qlin_matvec(dst, slice, type, n_cols, x, rows_per_expert);
}

static constexpr size_t kDenseLibWorkspace = (size_t)32 << 20; /* handed to the library GEMM */
static constexpr int kDenseMinTokens = 8;                     /* below this the vector-ALU kernel is faster than decode + GEMM */

int qlin_gemm_tokenmajor(float *Y, const void *W, uint32_t type, int n_cols, const float *X, int n_rows,
                         int n_tok, int out_stride, int x_stride) {
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || out_stride < n_rows || x_stride < n_cols) return fail(QLIN_ERR_ARG, "bad token count or stride");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!Y || !W || !X) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const size_t rb = row_size(type, n_cols);
    const void *dW;
    if (int rc = weights_on_device_locked(W, rb * (size_t)n_rows, g.w[0], &dW)) return rc;
    /* X and Y are staged densely (ldx = n_cols, ldy = n_rows); strides are applied by the copies */
    if (int rc = g.tmp[0].ensure((size_t)n_tok * n_cols * 4)) return rc;
    if (int rc = g.tmp[1].ensure((size_t)n_tok * n_rows * 4)) return rc;
    HIP_TRY(hipMemcpy2DAsync(g.tmp[0].p, (size_t)n_cols * 4, X, (size_t)x_stride * 4, (size_t)n_cols * 4,
                             (size_t)n_tok, hipMemcpyHostToDevice, g.stream));
    if (g.prefill_bf16 && n_tok >= 8 && n_cols % 8 == 0) {
        /* opted in: activations rounded to bf16 on the device, then the matrix-core route of
         * qlin_gemm_bf16_any_dev with internal scratch */
        const size_t ws_bytes = dense_gemm_weight_bytes(n_rows, n_cols) + ((size_t)32 << 20);
        if (int rc = g.tmp[2].ensure((size_t)n_tok * n_cols * 2)) return rc;
        if (int rc = g.tmp[3].ensure(ws_bytes)) return rc;
        HIP_TRY(launch_dequant_bf16(T_F32, g.tmp[0].p, (uint16_t *)g.tmp[2].p, n_tok, n_cols, (size_t)n_cols * 4, g.stream));
        const uint16_t *Xb = (const uint16_t *)g.tmp[2].p;
        float *Yd = (float *)g.tmp[1].p;
        const FusedTile tile = choose_fused_tile(type, n_rows, n_cols, n_tok, n_cols, true);
        if (type == T_Q4_K && n_tok <= kFewTokens) {
            HIP_TRY(launch_gemm_q4k_bf16(dW, Xb, Yd, n_rows, n_cols, n_tok, n_cols, n_rows, g.stream));
        } else if (tile != kFusedNone) {
            HIP_TRY(launch_fused_tile(tile, type, dW, Xb, Yd, n_rows, n_cols, n_tok, n_cols, n_rows, g.stream));
        } else {
            const uint16_t *Wd = (const uint16_t *)dW;
            if (type != T_BF16) {
                HIP_TRY(launch_dequant_bf16(type, dW, (uint16_t *)g.tmp[3].p, n_rows, n_cols, rb, g.stream));
                Wd = (const uint16_t *)g.tmp[3].p;
            }
            void *lib_ws = (char *)g.tmp[3].p + dense_gemm_weight_bytes(n_rows, n_cols);
            if (const char *err = launch_gemm_dense_bf16(Wd, Xb, Yd, n_rows, n_cols, n_tok, n_cols, n_rows, lib_ws,
                                                         (size_t)32 << 20, g.stream))
                return fail(QLIN_ERR_DEVICE, "dense bf16 GEMM: %s", err);
        }
    } else if (n_tok >= kDenseMinTokens) {
        /* exact weights, fp32 activations, fp32 accumulation on the matrix cores: bands of rows are decoded
         * to fp32 scratch (at most 512 MiB at a time) and multiplied by the library's dense fp32 GEMM */
        const size_t rows_in_512mib = (((size_t)512 << 20) / ((size_t)n_cols * 4)) & ~(size_t)255;
        const int band = (int)std::min<size_t>((size_t)n_rows, std::max<size_t>(256, rows_in_512mib));
        const size_t w_bytes = dense_gemm_weight_bytes_f32(band, n_cols);
        if (int rc = g.tmp[3].ensure(w_bytes + kDenseLibWorkspace)) return rc;
        float *Wf = (float *)g.tmp[3].p;
        void *lib_ws = (char *)g.tmp[3].p + w_bytes;
        for (int r0 = 0; r0 < n_rows; r0 += band) {
            const int nr = std::min(band, n_rows - r0);
            const uint8_t *Wb = (const uint8_t *)dW + (size_t)r0 * rb;
            const float *Wd = (const float *)Wb; /* fp32 weights are used where they are */
            if (type != T_F32) {
                HIP_TRY(launch_dequant(type, Wb, nullptr, nr, Wf, nr, n_cols, rb, g.stream));
                Wd = Wf;
            }
            float *Yd = (float *)g.tmp[1].p + r0;
            if (launch_gemm_dense(true, Wd, g.tmp[0].p, Yd, nr, n_cols, n_tok, n_cols, n_rows, lib_ws, kDenseLibWorkspace,
                                  g.stream) != nullptr) /* a shape the library has no kernel for */
                HIP_TRY(launch_gemm_f32(type, Wb, (const float *)g.tmp[0].p, Yd, nr, n_cols, n_tok, n_cols, n_rows, g.stream));
        }
    } else {
        HIP_TRY(launch_gemm_f32(type, dW, (const float *)g.tmp[0].p, (float *)g.tmp[1].p, n_rows, n_cols, n_tok,
                                n_cols, n_rows, g.stream));
    }
    HIP_TRY(hipMemcpy2DAsync(Y, (size_t)out_stride * 4, g.tmp[1].p, (size_t)n_rows * 4, (size_t)n_rows * 4,
                             (size_t)n_tok, hipMemcpyDeviceToHost, g.stream));
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

int qlin_set_dense_gemm_own(int enable) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    if (enable < 0 || enable > 2) return fail(QLIN_ERR_ARG, "0: vendor library, 1: own tile kernel, 2: vector-ALU kernel");
    g.dense_gemm_mode = enable;
    return QLIN_OK;
}

int qlin_set_prefill_matrix_cores(int enable) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    g.prefill_bf16 = enable != 0;
    return QLIN_OK;
}

int qlin_moe_ffn_token(float *out, const void *gate_exps, const void *up_exps, const void *down_exps,
                       uint32_t type, int n_embd, int n_ff, int n_expert, int top_k,
                       const float *router_logits, const float *x) {
    return qlin_moe_ffn_token_types(out, gate_exps, up_exps, down_exps, type, type, type, n_embd, n_ff, n_expert, top_k,
                                    router_logits, x);
}

int qlin_moe_ffn_token_types(float *out, const void *gate_exps, const void *up_exps, const void *down_exps,
                             uint32_t type_gate, uint32_t type_up, uint32_t type_down, int n_embd, int n_ff,
                             int n_expert, int top_k, const float *router_logits, const float *x) {
    if (int rc = check_linear_shape(type_gate, n_ff, n_embd)) return rc;
    if (int rc = check_linear_shape(type_up, n_ff, n_embd)) return rc;
    if (int rc = check_linear_shape(type_down, n_embd, n_ff)) return rc;
    if (n_expert <= 0 || top_k <= 0 || top_k > n_expert || top_k > 64 || n_expert > 8192)
        return fail(QLIN_ERR_ARG, "bad expert counts (n_expert %d, top_k %d)", n_expert, top_k);
    if (!out || !gate_exps || !up_exps || !down_exps || !router_logits || !x) return fail(QLIN_ERR_ARG, "null pointer");
    std::lock_guard<std::mutex> lk(g.mu);
    if (int rc = ensure_init_locked(0)) return rc;
    const size_t rb_g = row_size(type_gate, n_embd), rb_u = row_size(type_up, n_embd), rb_dn = row_size(type_down, n_ff);
    const void *dG, *dU, *dD;
    if (int rc = weights_on_device_locked(gate_exps, rb_g * (size_t)n_ff * n_expert, g.w[0], &dG)) return rc;
    if (int rc = weights_on_device_locked(up_exps, rb_u * (size_t)n_ff * n_expert, g.w[1], &dU)) return rc;
    if (int rc = weights_on_device_locked(down_exps, rb_dn * (size_t)n_embd * n_expert, g.w[2], &dD)) return rc;
    /* tmp[0]: logits | idx | w ; tmp[1]: gate ; tmp[2]: up ; tmp[3]: down out ; y[0]: accumulated out */
    const size_t off_idx = ((size_t)n_expert * 4 + 255) & ~(size_t)255;
    const size_t off_w = off_idx + 256;
    if (int rc = g.tmp[0].ensure(off_w + 256)) return rc;
    if (int rc = g.tmp[1].ensure((size_t)n_ff * 4)) return rc;
    if (int rc = g.tmp[2].ensure((size_t)n_ff * 4)) return rc;
    if (int rc = g.tmp[3].ensure((size_t)n_embd * 4)) return rc;
    if (int rc = g.y[0].ensure((size_t)n_embd * 4)) return rc;
    if (int rc = g.x.ensure((size_t)n_embd * 4)) return rc;
    uint8_t *t0 = (uint8_t *)g.tmp[0].p;
    int32_t *d_idx = (int32_t *)(t0 + off_idx);
    float *d_w = (float *)(t0 + off_w);
    HIP_TRY(hipMemcpyAsync(t0, router_logits, (size_t)n_expert * 4, hipMemcpyHostToDevice, g.stream));
    if (int rc = upload_locked(g.x.p, x, (size_t)n_embd * 4)) return rc;
    HIP_TRY(launch_moe_route((const float *)t0, 1, n_expert, top_k, d_idx, d_w, g.stream));
    int32_t h_idx[64];
    HIP_TRY(hipMemcpyAsync(h_idx, d_idx, (size_t)top_k * 4, hipMemcpyDeviceToHost, g.stream));
    if (int rc = finish_locked()) return rc;
    for (int k = 0; k < top_k; k++) {
        const int e = h_idx[k];
        if (e < 0 || e >= n_expert) return fail(QLIN_ERR_DEVICE, "router produced expert %d", e);
        const uint8_t *ge = (const uint8_t *)dG + (size_t)e * n_ff * rb_g;
        const uint8_t *ue = (const uint8_t *)dU + (size_t)e * n_ff * rb_u;
        const uint8_t *de = (const uint8_t *)dD + (size_t)e * n_embd * rb_dn;
        if (type_gate == type_up) { /* one launch: silu(gate x) * (up x) */
            const GemvJob gate_up = {{ge, ue, nullptr}, {(float *)g.tmp[1].p, nullptr, nullptr}, {n_ff, n_ff, 0}, 2, kSiluMul};
            HIP_TRY(dispatch_gemv_job(type_gate, gate_up, (const float *)g.x.p, n_embd, g.stream));
        } else {
            HIP_TRY(dispatch_gemv(type_gate, ge, (const float *)g.x.p, (float *)g.tmp[1].p, n_ff, n_embd, g.stream));
            HIP_TRY(dispatch_gemv(type_up, ue, (const float *)g.x.p, (float *)g.tmp[2].p, n_ff, n_embd, g.stream));
            HIP_TRY(launch_silu_mul((float *)g.tmp[1].p, (const float *)g.tmp[1].p, (const float *)g.tmp[2].p, n_ff, g.stream));
        }
        HIP_TRY(dispatch_gemv(type_down, de, (const float *)g.tmp[1].p, (float *)g.tmp[3].p, n_embd, n_ff, g.stream));
        HIP_TRY(launch_axpy_dev_weight((float *)g.y[0].p, (const float *)g.tmp[3].p, d_w, k, n_embd, k == 0, g.stream));
    }
    if (int rc = download_locked(out, g.y[0].p, (size_t)n_embd * 4)) return rc;
    if (int rc = finish_locked()) return rc;
    return QLIN_OK;
}

/* ------------------------------------------------------------------ device-resident */

void *qlin_dev_alloc(size_t n_bytes) {
    std::lock_guard<std::mutex> lk(g.mu);
    if (ensure_init_locked(0)) return nullptr;
    void *p = nullptr;
    if (hipMalloc(&p, n_bytes ? n_bytes : 1) != hipSuccess) {
        fail(QLIN_ERR_NOMEM, "hipMalloc of %zu bytes failed", n_bytes);
        return nullptr;
    }
    return p;
}

void qlin_dev_free(void *p) {
    if (p) (void)hipFree(p);
}

int qlin_dev_upload(void *dst_dev, const void *src_host, size_t n_bytes) {
    if (n_bytes == 0) return QLIN_OK;
    if (!dst_dev || !src_host) return fail(QLIN_ERR_ARG, "null pointer");
    HIP_TRY(hipMemcpy(dst_dev, src_host, n_bytes, hipMemcpyHostToDevice));
    return QLIN_OK;
}

int qlin_dev_download(void *dst_host, const void *src_dev, size_t n_bytes) {
    if (n_bytes == 0) return QLIN_OK;
    if (!dst_host || !src_dev) return fail(QLIN_ERR_ARG, "null pointer");
    HIP_TRY(hipMemcpy(dst_host, src_dev, n_bytes, hipMemcpyDeviceToHost));
    return QLIN_OK;
}

int qlin_dev_sync(void *stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return QLIN_OK;
}

int qlin_dequant_dev(uint32_t type, const void *W, float *out, int n_rows, int n_cols, void *stream) {
    if (!known_type(type)) return fail(QLIN_ERR_TYPE, "unsupported type %u", type);
    if (n_rows < 0 || n_cols < 0) return fail(QLIN_ERR_ARG, "negative size");
    if (n_rows == 0 || n_cols == 0) return QLIN_OK;
    if (!W || !out) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 2) || !aligned(out, 4)) return fail(QLIN_ERR_ARG, "W needs 2-byte, out 4-byte alignment");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_dequant(type, W, nullptr, 0, out, n_rows, n_cols, row_size(type, n_cols), (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_dequant_bf16_dev(uint32_t type, const void *W, uint16_t *out, int n_rows, int n_cols, void *stream) {
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!W || !out) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 16) || !aligned(out, 16)) return fail(QLIN_ERR_ARG, "W and out need 16-byte alignment");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_dequant_bf16(type, W, out, n_rows, n_cols, row_size(type, n_cols), (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_embed_rows_dev(uint32_t type, const void *table, int n_table_rows, const int32_t *row_ids, int n_ids,
                        float *out, int n_cols, void *stream) {
    if (!known_type(type)) return fail(QLIN_ERR_TYPE, "unsupported type %u", type);
    if (n_table_rows < 0 || n_ids < 0 || n_cols < 0) return fail(QLIN_ERR_ARG, "negative size");
    int be, bb;
    type_geometry(type, &be, &bb);
    if (n_cols % be) return fail(QLIN_ERR_ARG, "n_cols %d is not a whole number of %d-element blocks", n_cols, be);
    if (n_ids == 0 || n_cols == 0) return QLIN_OK;
    if (!table || !row_ids || !out) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(table, 2) || !aligned(row_ids, 4) || !aligned(out, 4)) return fail(QLIN_ERR_ARG, "misaligned pointer");
    if (int rc = init_once()) return rc;
    HIP_TRY(launch_dequant(type, table, row_ids, n_table_rows, out, n_ids, n_cols, row_size(type, n_cols),
                           (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemv_dev(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols, void *stream) {
    if (int rc = check_dev_gemv(type, n_rows, n_cols, W, x, y)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (int rc = init_once()) return rc;
    HIP_TRY(dispatch_gemv(type, W, x, y, n_rows, n_cols, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemv_add_dev(uint32_t type, const void *W, const float *x, float *y, int n_rows, int n_cols, void *stream) {
    if (int rc = check_dev_gemv(type, n_rows, n_cols, W, x, y)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (int rc = init_once()) return rc;
    HIP_TRY(dispatch_gemv_job(type, single_job(W, y, n_rows, kAdd), x, n_cols, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemv_silu_mul_dev(uint32_t type, const void *Wgate, const void *Wup, const float *x, float *out,
                           int n_rows, int n_cols, void *stream) {
    if (int rc = check_dev_gemv(type, n_rows, n_cols, Wgate, x, out)) return rc;
    if (n_rows == 0) return QLIN_OK;
    if (!Wup || !aligned(Wup, 2)) return fail(QLIN_ERR_ARG, "null or misaligned up matrix");
    if (int rc = init_once()) return rc;
    GemvJob job = {{Wgate, Wup, nullptr}, {out, nullptr, nullptr}, {n_rows, n_rows, 0}, 2, kSiluMul};
    HIP_TRY(dispatch_gemv_job(type, job, x, n_cols, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemv_multi_dev(uint32_t type, int n_mat, const void *const *W, float *const *y, const int *n_rows,
                        const float *x, int n_cols, void *stream) {
    if (n_mat < 1 || n_mat > 3 || !W || !y || !n_rows) return fail(QLIN_ERR_ARG, "1 to 3 matrices");
    GemvJob job = {{nullptr, nullptr, nullptr}, {nullptr, nullptr, nullptr}, {0, 0, 0}, n_mat, kStore};
    for (int m = 0; m < n_mat; m++) {
        if (int rc = check_dev_gemv(type, n_rows[m], n_cols, W[m], x, y[m])) return rc;
        job.W[m] = W[m];
        job.y[m] = y[m];
        job.n_rows[m] = n_rows[m];
    }
    if (job.total_rows() == 0) return QLIN_OK;
    if (int rc = init_once()) return rc;
    HIP_TRY(dispatch_gemv_job(type, job, x, n_cols, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemv_argmax_dev(uint32_t type, const void *W, const float *x, float *logits, void *result, int n_rows,
                         int n_cols, void *stream) {
    if (int rc = check_dev_gemv(type, n_rows, n_cols, W, x, logits)) return rc;
    if (n_rows == 0) return fail(QLIN_ERR_ARG, "argmax over no rows");
    if (!result || !aligned(result, 8)) return fail(QLIN_ERR_ARG, "result needs QLIN_ARGMAX_RESULT_BYTES bytes, 8-byte aligned");
    if (int rc = init_once()) return rc;
    HIP_TRY(dispatch_gemv(type, W, x, logits, n_rows, n_cols, (hipStream_t)stream));
    HIP_TRY(launch_argmax(logits, n_rows, (float *)result, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemm_f32_dev(uint32_t type, const void *W, const float *X, float *Y, int n_rows, int n_cols,
                      int n_tok, int ldx, int ldy, void *stream) {
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || ldx < n_cols || ldy < n_rows) return fail(QLIN_ERR_ARG, "bad token count or leading dimension");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!W || !X || !Y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 2) || !aligned(X, 4) || !aligned(Y, 4)) return fail(QLIN_ERR_ARG, "misaligned pointer");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_gemm_f32(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_gemm_bf16_dev(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                       int n_tok, int ldx, int ldy, void *stream) {
    if (type != T_Q4_K) return fail(QLIN_ERR_TYPE, "bf16 matrix-core GEMM takes Q4_K weights only (got %u)", type);
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || ldx < n_cols || ldy < n_rows) return fail(QLIN_ERR_ARG, "bad token count or leading dimension");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!W || !X || !Y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 16) || !aligned(X, 16) || !aligned(Y, 4) || ldx % 8)
        return fail(QLIN_ERR_ARG, "W and X need 16-byte alignment, Y 4-byte, ldx %% 8 == 0");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_gemm_q4k_bf16(W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
    return QLIN_OK;
}

size_t qlin_gemm_bf16_any_workspace_bytes(int n_rows, int n_cols) {
    if (n_rows <= 0 || n_cols <= 0) return 0;
    return dense_gemm_weight_bytes(n_rows, n_cols) + kDenseLibWorkspace;
}

int qlin_gemm_bf16_any_dev(uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                           int n_tok, int ldx, int ldy, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || ldx < n_cols || ldy < n_rows) return fail(QLIN_ERR_ARG, "bad token count or leading dimension");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!W || !X || !Y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 16) || !aligned(X, 16) || !aligned(Y, 4) || ldx % 8)
        return fail(QLIN_ERR_ARG, "W and X need 16-byte alignment, Y 4-byte, ldx %% 8 == 0");
    /* Q4_K, a few tokens: its few-token kernel (exact codes, no workspace) */
    const bool ws_ok = workspace && aligned(workspace, 256) && workspace_bytes >= qlin_gemm_bf16_any_workspace_bytes(n_rows, n_cols);
    if (type == T_Q4_K && n_tok <= kFewTokens)
        return qlin_gemm_bf16_dev(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, stream);
    /* a few tokens of a Q6_K, Q5_K, Q3_K, Q2_K or Q8_0 tensor: streamed once per eight tokens with exact codes
     * (14336 x 4096 Q6_K, 8 tokens: decode + library GEMM about 75 us) */
    {
        hipError_t e = hipSuccess;
        if (launch_gemm_kq_fewtok(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream, &e)) {
            if (e != hipSuccess) return fail(QLIN_ERR_DEVICE, "few-token GEMM launch failed: %s", hipGetErrorString(e));
            return QLIN_OK;
        }
    }
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    /* the formats with a tile kernel (gemm_kq_formats.h): decoded into the matrix operand inside the product, no workspace, in large or small
     * tiles by the shape - except where decoding once into the caller's workspace measured faster */
    /* (up to four tokens of the formats without a few-token kernel are faster one by one through the matvec below) */
    const bool matvec_first = (type == T_IQ4_NL || type == T_IQ4_XS || type == T_Q4_0) && n_tok <= kMatvecTokens && ws_ok;
    if (const FusedTile tile = matvec_first ? kFusedNone : choose_fused_tile(type, n_rows, n_cols, n_tok, ldx, ws_ok);
        tile != kFusedNone) {
        HIP_TRY(launch_fused_tile(tile, type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        return QLIN_OK;
    }
    if (!ws_ok)
        return fail(QLIN_ERR_ARG, "workspace must be 256-byte aligned and hold qlin_gemm_bf16_any_workspace_bytes(n_rows, n_cols) bytes");
    /* up to four tokens of any other block format: each through the matvec (exact weights; 14336 x 4096 IQ4_XS, four
     * tokens: 44 us against 95 us for decode + dense product), x widened to fp32 at the start of the workspace */
    const size_t x_span = (size_t)(n_tok - 1) * ldx + n_cols; /* elements of X from the first token's to the last's */
    if (n_tok <= kMatvecTokens && type != T_F32 && type != T_F16 && type != T_BF16 && x_span <= (size_t)INT_MAX &&
        x_span * sizeof(float) <= workspace_bytes) { /* a very wide ldx: the dense route below */
        float *xf = (float *)workspace;
        HIP_TRY(launch_dequant(T_BF16, X, nullptr, 0, xf, 1, (int)x_span, 0, (hipStream_t)stream));
        for (int t = 0; t < n_tok; t++)
            HIP_TRY(dispatch_gemv_job(type, single_job(W, Y + (size_t)t * ldy, n_rows), xf + (size_t)t * ldx, n_cols,
                                      (hipStream_t)stream));
        return QLIN_OK;
    }
    const uint16_t *Wd = (const uint16_t *)W; /* bf16 weights are used where they are */
    if (type != T_BF16) {
        HIP_TRY(launch_dequant_bf16(type, W, (uint16_t *)workspace, n_rows, n_cols, row_size(type, n_cols), (hipStream_t)stream));
        Wd = (const uint16_t *)workspace;
    }
    /* the dense product: the vendor library's kernel, or - where the library offers none for the shape, or
     * when asked for (QLIN_DENSE_GEMM=own, qlin_set_dense_gemm_own) - this library's own tile kernel
     * (gemm_dense_mfma.hip; K a multiple of 256) */
    const bool own_ok = n_cols % 256 == 0 && aligned(Wd, 16);
    const int mode = g.dense_gemm_mode;
    if (own_ok && mode == 1) {
        HIP_TRY(launch_gemm_dense_own(Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        return QLIN_OK;
    }
    void *lib_ws = (char *)workspace + dense_gemm_weight_bytes(n_rows, n_cols);
    const char *err = mode == 2 ? "switched off" : launch_gemm_dense_bf16(Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, lib_ws,
                                                                          kDenseLibWorkspace, (hipStream_t)stream);
    if (!err) return QLIN_OK;
    if (own_ok && mode != 2) { /* a shape the library has no kernel for */
        HIP_TRY(launch_gemm_dense_own(Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        return QLIN_OK;
    }
    /* neither takes the shape: the vector-ALU kernel on the weights as they came, the activations widened to fp32 a
     * band of tokens at a time in the library's part of the workspace */
    const size_t band = kDenseLibWorkspace / ((size_t)ldx * sizeof(float)); /* tokens widened at a time, gaps and all */
    if (band == 0) return fail(QLIN_ERR_DEVICE, "dense bf16 GEMM: %s", err);
    float *xf = (float *)lib_ws;
    for (size_t t0 = 0; t0 < (size_t)n_tok; t0 += band) {
        const int nt = (int)std::min<size_t>(band, (size_t)n_tok - t0);
        const size_t span = (size_t)(nt - 1) * ldx + n_cols;
        HIP_TRY(launch_dequant(T_BF16, X + t0 * ldx, nullptr, 0, xf, 1, (int)span, 0, (hipStream_t)stream));
        HIP_TRY(launch_gemm_f32(type, W, xf, Y + t0 * ldy, n_rows, n_cols, nt, ldx, ldy, (hipStream_t)stream));
    }
    return QLIN_OK;
}

int qlin_gemm_bf16_multi_dev(uint32_t type, int n_mat, const void *const *W, const uint16_t *X, float *const *Y,
                             const int *n_rows, int n_cols, int n_tok, int ldx, const int *ldy, void *workspace,
                             size_t workspace_bytes, void *stream) {
    if (n_mat < 1 || n_mat > 3) return fail(QLIN_ERR_ARG, "one to three tensors per call");
    if (!W || !Y || !n_rows || !ldy) return fail(QLIN_ERR_ARG, "null pointer");
    /* one launch where every tensor on its own would take the same tile kernel; the checks are those of the
     * single-tensor call, which a tensor that fails them goes through below to report it */
    bool together = n_mat > 1 && n_tok > 0 && X && aligned(X, 16) && ldx % 8 == 0 && ldx >= n_cols && n_tok > kFewTokens;
    FusedTile tile = kFusedNone;
    for (int i = 0; i < n_mat && together; i++) {
        const bool ws_ok = workspace && aligned(workspace, 256) &&
                           workspace_bytes >= qlin_gemm_bf16_any_workspace_bytes(n_rows[i], n_cols);
        together = n_rows[i] > 0 && W[i] && Y[i] && aligned(W[i], 16) && aligned(Y[i], 4) && ldy[i] >= n_rows[i] &&
                   n_cols > 0; /* the chooser checks format and row length */
        if (!together) break;
        const FusedTile mine = choose_fused_tile(type, n_rows[i], n_cols, n_tok, ldx, ws_ok);
        together = mine != kFusedNone && (i == 0 || mine == tile);
        tile = mine;
    }
    if (together) {
        {
            std::lock_guard<std::mutex> lk(g.mu);
            if (int rc = ensure_init_locked(0)) return rc;
        }
        if (tile == kFusedLarge)
            HIP_TRY(launch_gemm_kq_bf16_wave4_multi(type, n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        else
            HIP_TRY(launch_gemm_kq_bf16_wave4s_multi(type, n_mat, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        return QLIN_OK;
    }
    for (int i = 0; i < n_mat; i++)
        if (int rc = qlin_gemm_bf16_any_dev(type, W[i], X, Y[i], n_rows[i], n_cols, n_tok, ldx, ldy[i], workspace,
                                            workspace_bytes, stream))
            return rc;
    return QLIN_OK;
}

size_t qlin_gemm_f32_any_workspace_bytes(int n_rows, int n_cols) {
    if (n_rows <= 0 || n_cols <= 0) return 0;
    return dense_gemm_weight_bytes_f32(n_rows, n_cols) + kDenseLibWorkspace;
}

int qlin_gemm_f32_any_dev(uint32_t type, const void *W, const float *X, float *Y, int n_rows, int n_cols,
                          int n_tok, int ldx, int ldy, void *workspace, size_t workspace_bytes, void *stream) {
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || ldx < n_cols || ldy < n_rows) return fail(QLIN_ERR_ARG, "bad token count or leading dimension");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!W || !X || !Y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, type == T_F32 ? 4 : 2) || !aligned(X, 4) || !aligned(Y, 4)) return fail(QLIN_ERR_ARG, "misaligned pointer");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    if (n_tok < kDenseMinTokens) { /* a few tokens: the vector-ALU kernel, no workspace */
        HIP_TRY(launch_gemm_f32(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream));
        return QLIN_OK;
    }
    if (!workspace || !aligned(workspace, 256) || workspace_bytes < qlin_gemm_f32_any_workspace_bytes(n_rows, n_cols))
        return fail(QLIN_ERR_ARG, "workspace must be 256-byte aligned and hold qlin_gemm_f32_any_workspace_bytes(n_rows, n_cols) bytes");
    const float *Wd = (const float *)W; /* fp32 weights are used where they are */
    if (type != T_F32) {
        HIP_TRY(launch_dequant(type, W, nullptr, n_rows, (float *)workspace, n_rows, n_cols, row_size(type, n_cols),
                               (hipStream_t)stream));
        Wd = (const float *)workspace;
    }
    void *lib_ws = (char *)workspace + dense_gemm_weight_bytes_f32(n_rows, n_cols);
    if (launch_gemm_dense(true, Wd, X, Y, n_rows, n_cols, n_tok, ldx, ldy, lib_ws, kDenseLibWorkspace, (hipStream_t)stream) != nullptr)
        HIP_TRY(launch_gemm_f32(type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy, (hipStream_t)stream)); /* no library kernel for this shape */
    return QLIN_OK;
}

int qlin_moe_route_dev(const float *router_logits, int n_tok, int n_expert, int top_k, int32_t *expert_idx,
                       float *expert_w, void *stream) {
    if (n_tok < 0 || n_expert <= 0 || top_k <= 0 || top_k > n_expert || n_expert > 8192)
        return fail(QLIN_ERR_ARG, "bad routing shape");
    if (n_tok == 0) return QLIN_OK;
    if (!router_logits || !expert_idx || !expert_w) return fail(QLIN_ERR_ARG, "null pointer");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_moe_route(router_logits, n_tok, n_expert, top_k, expert_idx, expert_w, (hipStream_t)stream));
    return QLIN_OK;
}

size_t qlin_moe_workspace_bytes(int n_tok, int top_k, int n_embd, int n_ff, int n_expert) {
    return moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert);
}

static_assert(kMoeStaticScratchBytes == QLIN_MOE_STATIC_SCRATCH_BYTES, "the header states the size of the scratch");

static int check_moe_args(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate_exps,
                          const void *up_exps, const void *down_exps, const uint16_t *X, const int32_t *expert_idx,
                          const float *expert_w, float *out, int n_tok, int top_k, int n_embd, int n_ff, int n_expert) {
    if (int rc = check_linear_shape(type_gate, n_ff, n_embd)) return rc;
    if (int rc = check_linear_shape(type_up, n_ff, n_embd)) return rc;
    if (int rc = check_linear_shape(type_down, n_embd, n_ff)) return rc;
    if (n_embd % 8 || n_ff % 8) return fail(QLIN_ERR_ARG, "n_embd and n_ff must be multiples of 8");
    if (n_tok < 0 || n_expert <= 0 || top_k <= 0 || top_k > n_expert) return fail(QLIN_ERR_ARG, "bad MoE shape");
    if (n_expert > 4096) return fail(QLIN_ERR_ARG, "grouped MoE FFN handles at most 4096 experts (got %d)", n_expert);
    if ((long long)n_tok * top_k > (1 << 24))
        return fail(QLIN_ERR_ARG, "grouped MoE FFN handles at most 2^24 (token, expert) pairs per call");
    if (n_tok == 0) return QLIN_OK;
    if (!gate_exps || !up_exps || !down_exps || !X || !expert_idx || !expert_w || !out)
        return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(gate_exps, 16) || !aligned(up_exps, 16) || !aligned(down_exps, 16) || !aligned(X, 16) || !aligned(out, 16))
        return fail(QLIN_ERR_ARG, "misaligned pointer (16 bytes)");
    return QLIN_OK;
}

int qlin_moe_ffn_types_dev(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate_exps,
                           const void *up_exps, const void *down_exps, const uint16_t *X, const int32_t *expert_idx,
                           const float *expert_w, float *out, int n_tok, int top_k, int n_embd, int n_ff, int n_expert,
                           void *workspace, void *stream) {
    if (int rc = check_moe_args(type_gate, type_up, type_down, gate_exps, up_exps, down_exps, X, expert_idx, expert_w, out,
                                n_tok, top_k, n_embd, n_ff, n_expert))
        return rc;
    if (n_tok == 0) return QLIN_OK;
    if (!workspace) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(workspace, 256)) return fail(QLIN_ERR_ARG, "misaligned pointer (workspace: 256 bytes)");
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    HIP_TRY(launch_moe_ffn(type_gate, type_up, type_down, gate_exps, up_exps, down_exps, X, expert_idx, expert_w, out,
                           n_tok, top_k, n_embd, n_ff, n_expert, g.n_cu, workspace, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_moe_ffn_static_dev(uint32_t type_gate, uint32_t type_up, uint32_t type_down, const void *gate_exps,
                            const void *up_exps, const void *down_exps, const uint16_t *X, const int32_t *expert_idx,
                            const float *expert_w, float *out, int n_tok, int top_k, int n_embd, int n_ff, int n_expert,
                            void *stream) {
    if (int rc = check_moe_args(type_gate, type_up, type_down, gate_exps, up_exps, down_exps, X, expert_idx, expert_w, out,
                                n_tok, top_k, n_embd, n_ff, n_expert))
        return rc;
    if (n_tok == 0) return QLIN_OK;
    const size_t need = moe_workspace_bytes(n_tok, top_k, n_embd, n_ff, n_expert);
    if (need > (size_t)QLIN_MOE_STATIC_SCRATCH_BYTES)
        return fail(QLIN_ERR_ARG, "this shape needs %zu bytes of scratch, the built-in scratch holds %zu: use qlin_moe_ffn_types_dev "
                                  "with a workspace", need, (size_t)QLIN_MOE_STATIC_SCRATCH_BYTES);
    int device, n_cu;
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (!g.ready) /* initialising would allocate (stream, events): that is qlin_init's job, not this call's */
            return fail(QLIN_ERR_DEVICE, "qlin_init() must have run before qlin_moe_ffn_static_dev");
        device = g.device;
        n_cu = g.n_cu;
    }
    HIP_TRY(launch_moe_ffn_static(type_gate, type_up, type_down, gate_exps, up_exps, down_exps, X, expert_idx, expert_w, out,
                                  n_tok, top_k, n_embd, n_ff, n_expert, device, n_cu, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_moe_ffn_dev(uint32_t type, const void *gate_exps, const void *up_exps, const void *down_exps,
                     const uint16_t *X, const int32_t *expert_idx, const float *expert_w, float *out,
                     int n_tok, int top_k, int n_embd, int n_ff, int n_expert, void *workspace, void *stream) {
    return qlin_moe_ffn_types_dev(type, type, type, gate_exps, up_exps, down_exps, X, expert_idx, expert_w, out, n_tok,
                                  top_k, n_embd, n_ff, n_expert, workspace, stream);
}

int qlin_probe_mfma_bf16(int iters, void *stream, double *flops) {
    if (iters <= 0 || iters > (1 << 22) || !flops) return fail(QLIN_ERR_ARG, "iters must be in 1..2^22 and flops non-null");
    if (int rc = init_once()) return rc;
    HIP_TRY(launch_probe_mfma(iters, g.n_cu, (hipStream_t)stream, flops));
    return QLIN_OK;
}

int qlin_probe_clocks(void *stream, double *shader_mhz) {
    if (!shader_mhz) return fail(QLIN_ERR_ARG, "null pointer");
    if (int rc = init_once()) return rc;
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    uint64_t c[2] = {0, 0};
    HIP_TRY(read_probe_clocks(c));
    if (c[1] == 0) return fail(QLIN_ERR_ARG, "qlin_probe_mfma_bf16 has not run");
    *shader_mhz = (double)c[0] * 100.0 / (double)c[1];
    return QLIN_OK;
}

int qlin_probe_gemm_route(uint32_t type, int n_rows, int n_cols, int n_tok, int ldx, int have_workspace) {
    return (int)choose_fused_tile(type, n_rows, n_cols, n_tok, ldx, have_workspace != 0);
}

int qlin_probe_gemm_tile(int tile, uint32_t type, const void *W, const uint16_t *X, float *Y, int n_rows, int n_cols,
                         int n_tok, int ldx, int ldy, void *stream) {
    if (tile < 0 || tile > 1) return fail(QLIN_ERR_ARG, "tile: 0 (256 x 128) or 1 (128 x 64)");
    if (!gemm_kq_wave4_covers(type)) return fail(QLIN_ERR_TYPE, "no fused tile kernel for type %u", type);
    if (int rc = check_linear_shape(type, n_rows, n_cols)) return rc;
    if (n_tok < 0 || ldx < n_cols || ldy < n_rows || n_cols % 256 || ldx >= (1 << 22))
        return fail(QLIN_ERR_ARG, "bad token count, leading dimension or row length");
    if (n_rows == 0 || n_tok == 0) return QLIN_OK;
    if (!W || !X || !Y) return fail(QLIN_ERR_ARG, "null pointer");
    if (!aligned(W, 16) || !aligned(X, 16) || !aligned(Y, 4) || ldx % 8)
        return fail(QLIN_ERR_ARG, "W and X need 16-byte alignment, Y 4-byte, ldx %% 8 == 0");
    if (int rc = init_once()) return rc;
    HIP_TRY(launch_fused_tile(tile == 0 ? kFusedLarge : kFusedSmall, type, W, X, Y, n_rows, n_cols, n_tok, ldx, ldy,
                              (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_probe_hbm_read(const void *buf, size_t n_bytes, void *stream) {
    if (!buf || n_bytes < 16 || ((uintptr_t)buf & 15)) return fail(QLIN_ERR_ARG, "buffer must be 16-byte aligned and at least 16 bytes");
    if (n_bytes / 16 / 2048 > 0x7fffffffu) return fail(QLIN_ERR_ARG, "buffer too large for one launch");
    if (int rc = init_once()) return rc;
    HIP_TRY(launch_probe_read(buf, n_bytes, (hipStream_t)stream));
    return QLIN_OK;
}

int qlin_timer_begin(void *stream) {
    {
        std::lock_guard<std::mutex> lk(g.mu);
        if (int rc = ensure_init_locked(0)) return rc;
    }
    if (!t_timer.ev0) {
        HIP_TRY(hipEventCreate(&t_timer.ev0));
        HIP_TRY(hipEventCreate(&t_timer.ev1));
    }
    HIP_TRY(hipEventRecord(t_timer.ev0, (hipStream_t)stream));
    t_timer.begun = true;
    return QLIN_OK;
}

int qlin_timer_end(void *stream, float *ms) {
    if (!t_timer.begun) return fail(QLIN_ERR_ARG, "qlin_timer_begin was not called on this thread");
    if (!ms) return fail(QLIN_ERR_ARG, "null pointer");
    HIP_TRY(hipEventRecord(t_timer.ev1, (hipStream_t)stream));
    HIP_TRY(hipEventSynchronize(t_timer.ev1));
    HIP_TRY(hipEventElapsedTime(ms, t_timer.ev0, t_timer.ev1));
    return QLIN_OK;
}

}  // extern "C"
