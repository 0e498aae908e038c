/*
 * gguf_upload.hip - GGUF file -> HBM: the tensor table of a model file and its tensor bytes in
 * device memory, without the reference's loader in between.
 *
 * The file format as the reference reads it (common/gguf_loader.h:343-411): magic "GGUF", version
 * 2 or 3, tensor and key/value counts, the key/value pairs (typed scalars, strings, arrays), the
 * tensor infos (name, up to 4 dims, ggml type, offset into the data section) and, at the next
 * multiple of general.alignment (default 32), the data section. A tensor's size is
 * ceil(elements / block_elems) * block_bytes (:520-532).
 *
 * Where the reference maps the whole file and touches every page (MAP_POPULATE, :443-451) and
 * its GPU runners then copy tensor by tensor, this loader
 *   - maps the file lazily, only to read the header and to give every tensor a stable host
 *     address (the key under which host-pointer entry points find the device copy),
 *   - allocates ONE device block for the whole data section (weights stay in wire format, so the
 *     file's own layout is the HBM layout) and streams the section into it with pread() into two
 *     pinned staging buffers that alternate between disk reads and asynchronous copies,
 *   - registers [host data base, +size) -> device block, so that tf_load_tensor-style code can keep
 *     passing `mapping + offset` pointers and never causes another upload.
 * Every length read from the file is checked against the file size before it is used.
 */
#include "../../include/qlinear.h"

#include <hip/hip_runtime.h>

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {
int set_error(int code, const char *fmt, ...); /* qlin_api.hip: records the text qlin_last_error() returns */
}

namespace {

using qlin::set_error;

enum : uint32_t { V_U8, V_I8, V_U16, V_I16, V_U32, V_I32, V_F32, V_BOOL, V_STR, V_ARR, V_U64, V_I64, V_F64 };

size_t scalar_size(uint32_t t) {
    switch (t) {
    case V_U8: case V_I8: case V_BOOL: return 1;
    case V_U16: case V_I16: return 2;
    case V_U32: case V_I32: case V_F32: return 4;
    case V_U64: case V_I64: case V_F64: return 8;
    default: return 0;
    }
}

/* elements and bytes per block of every ggml type id a file may carry (common/gguf_loader.h:184-223);
 * the types without a decoder here only need their size */
bool storage_geometry(uint32_t t, int *be, int *bb) {
    if (qlin::type_geometry(t, be, bb)) return true;
    switch (t) {
    case 9: *be = 32; *bb = 36; return true;                 /* Q8_1 */
    case 15: *be = 256; *bb = 292; return true;              /* Q8_K */
    case 24: *be = 1; *bb = 1; return true;                  /* I8 */
    case 25: *be = 1; *bb = 2; return true;                  /* I16 */
    case 26: *be = 1; *bb = 4; return true;                  /* I32 */
    case 27: case 28: *be = 1; *bb = 8; return true;         /* I64, F64 */
    case 31: case 32: case 33: *be = 32; *bb = 18; return true; /* repacked Q4_0 variants */
    default: return false;
    }
}

struct Kv {
    std::string key;
    uint32_t type = 0;
    uint64_t bits = 0;        /* scalar value, zero-extended little-endian bytes */
    std::string str;          /* V_STR */
    uint32_t arr_type = 0;    /* V_ARR */
    uint64_t arr_n = 0;
    size_t arr_off = 0;       /* file offset of the first array element */
};

struct Tensor {
    std::string name;
    uint32_t n_dims = 0;
    uint64_t dims[4] = {0, 0, 0, 0};
    uint32_t type = 0;
    uint64_t offset = 0;
    size_t bytes = 0;
};

/* bounds-checked reader over the mapped file */
struct Cursor {
    const uint8_t *base;
    size_t size, pos;
    bool ok = true;
    template <typename T> T get() {
        T v{};
        if (!ok || size - pos < sizeof(T)) { ok = false; return v; }
        memcpy(&v, base + pos, sizeof(T));
        pos += sizeof(T);
        return v;
    }
    std::string str() {
        const uint64_t n = get<uint64_t>();
        if (!ok || n > size - pos) { ok = false; return std::string(); }
        std::string s(reinterpret_cast<const char *>(base + pos), (size_t)n);
        pos += (size_t)n;
        return s;
    }
    void skip(uint64_t n) {
        if (!ok || n > size - pos) { ok = false; return; }
        pos += (size_t)n;
    }
};

}  // namespace

struct qlin_gguf {
    int fd = -1;
    void *map = nullptr;
    size_t file_size = 0;
    uint32_t version = 0, alignment = 32;
    size_t data_offset = 0, data_size = 0;
    std::vector<Kv> kv;
    std::vector<Tensor> tensors;
    void *dev = nullptr; /* the data section in HBM, once uploaded */
    bool registered = false;
};

namespace {

bool read_value(Cursor &c, Kv &kv, uint32_t type) {
    kv.type = type;
    if (const size_t n = scalar_size(type)) {
        if (c.size - c.pos < n) return c.ok = false;
        memcpy(&kv.bits, c.base + c.pos, n);
        c.pos += n;
        return c.ok;
    }
    if (type == V_STR) {
        kv.str = c.str();
        return c.ok;
    }
    if (type == V_ARR) {
        kv.arr_type = c.get<uint32_t>();
        kv.arr_n = c.get<uint64_t>();
        kv.arr_off = c.pos;
        if (kv.arr_type == V_STR) {
            for (uint64_t i = 0; c.ok && i < kv.arr_n; i++) c.skip(c.get<uint64_t>());
        } else {
            const size_t es = scalar_size(kv.arr_type);
            if (es == 0 || kv.arr_n > (c.size - c.pos) / es) return c.ok = false;
            c.skip(kv.arr_n * es);
        }
        return c.ok;
    }
    return c.ok = false;
}

int parse(qlin_gguf *g) {
    Cursor c{static_cast<const uint8_t *>(g->map), g->file_size, 0};
    if (c.get<uint32_t>() != 0x46554747u || !c.ok) return set_error(QLIN_ERR_ARG, "gguf: bad magic");
    g->version = c.get<uint32_t>();
    if (!c.ok || (g->version != 2 && g->version != 3)) return set_error(QLIN_ERR_ARG, "gguf: unsupported version %u", g->version);
    const uint64_t n_tensors = c.get<uint64_t>(), n_kv = c.get<uint64_t>();
    /* a key/value pair takes at least 12 bytes, a tensor info at least 24 */
    if (!c.ok || n_kv > g->file_size / 12 || n_tensors > g->file_size / 24)
        return set_error(QLIN_ERR_ARG, "gguf: counts exceed the file size");
    g->kv.resize((size_t)n_kv);
    for (auto &kv : g->kv) {
        kv.key = c.str();
        const uint32_t t = c.get<uint32_t>();
        if (!c.ok || !read_value(c, kv, t)) return set_error(QLIN_ERR_ARG, "gguf: truncated or malformed key/value section");
    }
    for (const auto &kv : g->kv)
        if (kv.key == "general.alignment" && kv.type == V_U32) g->alignment = (uint32_t)kv.bits;
    if (g->alignment == 0) return set_error(QLIN_ERR_ARG, "gguf: alignment 0");
    g->tensors.resize((size_t)n_tensors);
    for (auto &t : g->tensors) {
        t.name = c.str();
        t.n_dims = c.get<uint32_t>();
        if (!c.ok || t.n_dims > 4) return set_error(QLIN_ERR_ARG, "gguf: tensor with %u dimensions", t.n_dims);
        for (uint32_t d = 0; d < t.n_dims; d++) t.dims[d] = c.get<uint64_t>();
        t.type = c.get<uint32_t>();
        t.offset = c.get<uint64_t>();
        if (!c.ok) return set_error(QLIN_ERR_ARG, "gguf: truncated tensor table");
    }
    g->data_offset = (c.pos + g->alignment - 1) / g->alignment * g->alignment;
    /* a file without tensors may end before the aligned start of its (empty) data section */
    const size_t room = g->data_offset <= g->file_size ? g->file_size - g->data_offset : 0;
    size_t end_max = 0;
    for (auto &t : g->tensors) {
        int be, bb;
        if (!storage_geometry(t.type, &be, &bb)) return set_error(QLIN_ERR_TYPE, "gguf: tensor '%s' has unknown type %u", t.name.c_str(), t.type);
        unsigned __int128 n = 1;
        for (uint32_t d = 0; d < t.n_dims; d++) {
            n *= t.dims[d];
            if (n > ((unsigned __int128)1 << 62)) return set_error(QLIN_ERR_ARG, "gguf: tensor '%s' is too large", t.name.c_str());
        }
        const uint64_t elems = (uint64_t)n;
        t.bytes = (size_t)((elems + be - 1) / be) * (size_t)bb;
        if (t.offset > room || t.bytes > room - t.offset)
            return set_error(QLIN_ERR_ARG, "gguf: tensor '%s' lies outside the file", t.name.c_str());
        if (t.offset + t.bytes > end_max) end_max = t.offset + t.bytes;
    }
    g->data_size = end_max;
    return QLIN_OK;
}

const Kv *kv_at(const qlin_gguf *g, int i) {
    return (g && i >= 0 && (size_t)i < g->kv.size()) ? &g->kv[(size_t)i] : nullptr;
}

}  // namespace

extern "C" {

int qlin_gguf_open(const char *path, qlin_gguf **out) {
    if (!path || !out) return set_error(QLIN_ERR_ARG, "null pointer");
    *out = nullptr;
    qlin_gguf *g = new qlin_gguf();
    g->fd = open(path, O_RDONLY);
    struct stat st;
    if (g->fd < 0 || fstat(g->fd, &st) != 0 || st.st_size < 24) {
        const int rc = set_error(QLIN_ERR_ARG, "gguf: cannot open %s (or shorter than a header)", path);
        qlin_gguf_close(g);
        return rc;
    }
    g->file_size = (size_t)st.st_size;
    g->map = mmap(nullptr, g->file_size, PROT_READ, MAP_PRIVATE, g->fd, 0);
    if (g->map == MAP_FAILED) {
        g->map = nullptr;
        const int rc = set_error(QLIN_ERR_NOMEM, "gguf: cannot map %s", path);
        qlin_gguf_close(g);
        return rc;
    }
    if (const int rc = parse(g)) {
        qlin_gguf_close(g);
        return rc;
    }
    *out = g;
    return QLIN_OK;
}

void qlin_gguf_close(qlin_gguf *g) {
    if (!g) return;
    if (g->registered) (void)qlin_weight_unregister(static_cast<const uint8_t *>(g->map) + g->data_offset);
    else if (g->dev) (void)hipFree(g->dev);
    if (g->map) munmap(g->map, g->file_size);
    if (g->fd >= 0) close(g->fd);
    delete g;
}

uint32_t qlin_gguf_version(const qlin_gguf *g) { return g ? g->version : 0; }
uint32_t qlin_gguf_alignment(const qlin_gguf *g) { return g ? g->alignment : 0; }
size_t qlin_gguf_data_offset(const qlin_gguf *g) { return g ? g->data_offset : 0; }
size_t qlin_gguf_data_size(const qlin_gguf *g) { return g ? g->data_size : 0; }
int qlin_gguf_n_tensors(const qlin_gguf *g) { return g ? (int)g->tensors.size() : 0; }
int qlin_gguf_n_kv(const qlin_gguf *g) { return g ? (int)g->kv.size() : 0; }

int qlin_gguf_find_tensor(const qlin_gguf *g, const char *name) {
    if (!g || !name) return -1;
    for (size_t i = 0; i < g->tensors.size(); i++)
        if (g->tensors[i].name == name) return (int)i;
    return -1;
}

int qlin_gguf_tensor_info(const qlin_gguf *g, int i, const char **name, uint32_t *ggml_type, int *n_dims,
                          uint64_t dims[4], uint64_t *offset, size_t *n_bytes) {
    if (!g || i < 0 || (size_t)i >= g->tensors.size()) return set_error(QLIN_ERR_ARG, "gguf: tensor index %d out of range", i);
    const Tensor &t = g->tensors[(size_t)i];
    if (name) *name = t.name.c_str();
    if (ggml_type) *ggml_type = t.type;
    if (n_dims) *n_dims = (int)t.n_dims;
    if (dims) memcpy(dims, t.dims, sizeof(t.dims));
    if (offset) *offset = t.offset;
    if (n_bytes) *n_bytes = t.bytes;
    return QLIN_OK;
}

const void *qlin_gguf_tensor_host(const qlin_gguf *g, int i) {
    if (!g || i < 0 || (size_t)i >= g->tensors.size()) return nullptr;
    return static_cast<const uint8_t *>(g->map) + g->data_offset + g->tensors[(size_t)i].offset;
}

const void *qlin_gguf_tensor_dev(const qlin_gguf *g, int i) {
    if (!g || !g->dev || i < 0 || (size_t)i >= g->tensors.size()) return nullptr;
    return static_cast<const uint8_t *>(g->dev) + g->tensors[(size_t)i].offset;
}

int qlin_gguf_find_key(const qlin_gguf *g, const char *key) {
    if (!g || !key) return -1;
    for (size_t i = 0; i < g->kv.size(); i++)
        if (g->kv[i].key == key) return (int)i;
    return -1;
}

const char *qlin_gguf_key(const qlin_gguf *g, int i) {
    const Kv *kv = kv_at(g, i);
    return kv ? kv->key.c_str() : nullptr;
}

int qlin_gguf_value_type(const qlin_gguf *g, int i) {
    const Kv *kv = kv_at(g, i);
    return kv ? (int)kv->type : -1;
}

/* numeric scalars of any integer width, sign- or zero-extended; bool as 0/1 */
int qlin_gguf_get_i64(const qlin_gguf *g, int i, int64_t *out) {
    const Kv *kv = kv_at(g, i);
    if (!kv || !out) return set_error(QLIN_ERR_ARG, "gguf: no such key");
    switch (kv->type) {
    case V_U8: case V_BOOL: *out = (uint8_t)kv->bits; return QLIN_OK;
    case V_I8: *out = (int8_t)kv->bits; return QLIN_OK;
    case V_U16: *out = (uint16_t)kv->bits; return QLIN_OK;
    case V_I16: *out = (int16_t)kv->bits; return QLIN_OK;
    case V_U32: *out = (uint32_t)kv->bits; return QLIN_OK;
    case V_I32: *out = (int32_t)kv->bits; return QLIN_OK;
    case V_U64: case V_I64: *out = (int64_t)kv->bits; return QLIN_OK;
    default: return set_error(QLIN_ERR_TYPE, "gguf: key '%s' is not an integer", kv->key.c_str());
    }
}

int qlin_gguf_get_f64(const qlin_gguf *g, int i, double *out) {
    const Kv *kv = kv_at(g, i);
    if (!kv || !out) return set_error(QLIN_ERR_ARG, "gguf: no such key");
    if (kv->type == V_F32) {
        float f;
        memcpy(&f, &kv->bits, 4);
        *out = f;
        return QLIN_OK;
    }
    if (kv->type == V_F64) {
        memcpy(out, &kv->bits, 8);
        return QLIN_OK;
    }
    int64_t v;
    if (qlin_gguf_get_i64(g, i, &v) != QLIN_OK) return set_error(QLIN_ERR_TYPE, "gguf: key '%s' is not a number", kv->key.c_str());
    *out = (double)v;
    return QLIN_OK;
}

const char *qlin_gguf_get_str(const qlin_gguf *g, int i) {
    const Kv *kv = kv_at(g, i);
    return (kv && kv->type == V_STR) ? kv->str.c_str() : nullptr;
}

int qlin_gguf_get_array(const qlin_gguf *g, int i, uint32_t *elem_type, uint64_t *n, const void **first) {
    const Kv *kv = kv_at(g, i);
    if (!kv || kv->type != V_ARR) return set_error(QLIN_ERR_TYPE, "gguf: not an array");
    if (elem_type) *elem_type = kv->arr_type;
    if (n) *n = kv->arr_n;
    if (first) *first = static_cast<const uint8_t *>(g->map) + kv->arr_off;
    return QLIN_OK;
}

int qlin_gguf_upload(qlin_gguf *g) {
    if (!g) return set_error(QLIN_ERR_ARG, "null pointer");
    if (g->dev) return QLIN_OK;
    if (g->data_size == 0) return QLIN_OK;
    if (const int rc = qlin_init(0)) return rc;
    void *dev = nullptr;
    if (hipMalloc(&dev, g->data_size + 256) != hipSuccess) /* same slack as qlin_weight_register */ return set_error(QLIN_ERR_NOMEM, "gguf: hipMalloc of %zu bytes failed", g->data_size);
    /* two pinned staging buffers: one is filled from the file while the other is in flight */
    const size_t kStage = (size_t)64 << 20;
    const size_t stage = g->data_size < kStage ? g->data_size : kStage;
    void *pin[2] = {nullptr, nullptr};
    hipStream_t s = nullptr;
    hipEvent_t done[2] = {nullptr, nullptr};
    int rc = QLIN_OK;
    auto hip_ok = [&](hipError_t e, const char *what) {
        if (e != hipSuccess && rc == QLIN_OK) rc = set_error(QLIN_ERR_DEVICE, "gguf: %s: %s", what, hipGetErrorString(e));
        return e == hipSuccess;
    };
    if (hip_ok(hipStreamCreate(&s), "stream")) {
        for (int b = 0; b < 2 && rc == QLIN_OK; b++) {
            hip_ok(hipHostMalloc(&pin[b], stage, hipHostMallocDefault), "pinned buffer");
            hip_ok(hipEventCreate(&done[b]), "event");
        }
        size_t off = 0;
        for (int turn = 0; rc == QLIN_OK && off < g->data_size; turn++) {
            const int b = turn & 1;
            if (turn >= 2 && !hip_ok(hipEventSynchronize(done[b]), "wait")) break;
            const size_t n = g->data_size - off < stage ? g->data_size - off : stage;
            size_t got = 0;
            while (got < n) {
                const ssize_t r = pread(g->fd, static_cast<uint8_t *>(pin[b]) + got, n - got, (off_t)(g->data_offset + off + got));
                if (r <= 0) { rc = set_error(QLIN_ERR_ARG, "gguf: read failed at offset %zu", g->data_offset + off + got); break; }
                got += (size_t)r;
            }
            if (rc != QLIN_OK) break;
            if (!hip_ok(hipMemcpyAsync(static_cast<uint8_t *>(dev) + off, pin[b], n, hipMemcpyHostToDevice, s), "copy")) break;
            hip_ok(hipEventRecord(done[b], s), "event record");
            off += n;
        }
        hip_ok(hipStreamSynchronize(s), "sync");
    }
    for (int b = 0; b < 2; b++) {
        if (pin[b]) (void)hipHostFree(pin[b]);
        if (done[b]) (void)hipEventDestroy(done[b]);
    }
    if (s) (void)hipStreamDestroy(s);
    if (rc != QLIN_OK) {
        (void)hipFree(dev);
        return rc;
    }
    g->dev = dev;
    /* host-pointer entry points that are handed `mapping + offset` now find the device copy */
    if (qlin_weight_adopt(static_cast<const uint8_t *>(g->map) + g->data_offset, g->data_size, dev) == QLIN_OK)
        g->registered = true;
    return QLIN_OK;
}

}  // extern "C"
