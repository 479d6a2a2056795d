/*
 * Host side of the C ABI declared in include/eri_optim8.h: device storage over the HIP runtime,
 * construction and self-check of the quantisation tables, validation and upload of the launch
 * table, and the step dispatch.  No torch, no CUDA shim; the only dependency is libamdhip64.
 */
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <mutex>
#include <string>
#include <vector>

#include "eri_adam8_device.h"
#include "eri_dynamic_maps.inc"

namespace {

thread_local std::string g_err;

int fail(int code, const std::string &msg) {
    g_err = msg;
    return code;
}

int hip_fail(hipError_t e, const char *what) {
    g_err = std::string(what) + ": " + hipGetErrorString(e);
    (void)hipGetLastError(); // reported here: the runtime's own record must not surface in the caller's next HIP call
    return (int)e;
}

#define ERI_HIP(call)                                        \
    do {                                                     \
        hipError_t e_ = (call);                              \
        if (e_ != hipSuccess) return hip_fail(e_, #call);    \
    } while (0)

inline float bits_to_float(uint32_t u) {
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// ---------------------------------------------------------------------------------------------
// quantisation tables
// ---------------------------------------------------------------------------------------------

struct Tables {
    float map_s[256], map_u[256];
    float mid_s[256], mid_u[256]; // 255 midpoints + inf
    std::vector<unsigned char> image;
    bool ok = false;
    std::string why;
};

uint32_t count_below(const float *mid, float x) { // the definition the slots must reproduce
    uint32_t n = 0;
    for (int j = 0; j < 255; ++j) n += (x > mid[j]) ? 1u : 0u;
    return n;
}

/* binary32 -> binary16 bit pattern, rounded toward zero (what v_cvt_pkrtz_f16_f32 does). */
uint16_t half_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t abs = u & 0x7fffffffu;
    if (abs > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);  // NaN
    if (abs == 0x7f800000u) return (uint16_t)(sign | 0x7c00u); // infinity stays infinity
    if (abs >= 0x477fe000u) return (uint16_t)(sign | 0x7bffu); // everything from 65504 up truncates to it
    const int exp = (int)(abs >> 23) - 127;
    if (exp < -24) return (uint16_t)sign;                      // below the smallest denormal
    const uint32_t mant = (abs & 0x7fffffu) | 0x800000u;
    if (exp < -14) return (uint16_t)(sign | (mant >> (13 + (-14 - exp)))); // denormal
    return (uint16_t)(sign | (((uint32_t)(exp + 15) << 10) + ((mant >> 13) - 0x400u)));
}

/*
 * Fills the slot table of one map.  `drop` low bits of the half pattern are ignored, `mask` is
 * applied first (it removes the sign for the unsigned map), `stride` bytes separate slots.
 * For each sign the magnitudes 0 .. kKeyScale are walked as bit patterns (which order floats of one
 * sign); every maximal run of magnitudes that convert into the same slot gives the slot's extreme
 * scaled quotients, and the slot is accepted only if at most one scaled midpoint lies between them.
 */
bool build_slots(const float *mid, uint32_t drop, uint32_t mask, uint32_t stride, uint32_t count,
                 unsigned char *out, std::string &why) {
    float smid[255];
    for (int j = 0; j < 255; ++j) smid[j] = mid[j] * eri::kKeyScale; // exact: power of two, no underflow
    const float inf = std::numeric_limits<float>::infinity();
    for (uint32_t k = 0; k < count; ++k) {
        eri::KeySlot s;
        s.lo = 0;
        s.mid = inf; // NaN and unreachable patterns answer code 0
        std::memcpy(out + (size_t)k * stride, &s, sizeof s);
    }
    uint32_t top_bits;
    std::memcpy(&top_bits, &eri::kKeyScale, 4);
    const int signs = (mask & 0x8000u) ? 2 : 1;
    for (int sg = 0; sg < signs; ++sg) {
        const uint32_t sign = sg ? 0x80000000u : 0u;
        auto value = [&](uint32_t mag) { return bits_to_float(mag | sign); };
        auto slot_of = [&](uint32_t mag) { return (uint32_t)((half_bits(value(mag)) & mask) >> drop); };
        uint32_t b_lo = 0;
        while (b_lo <= top_bits) {
            const uint32_t k = slot_of(b_lo);
            uint32_t a = b_lo, b = top_bits + 1; // slot_of(a) == k; b is past the run or past the range
            if (slot_of(top_bits) == k) a = top_bits;
            else {
                b = top_bits;
                while (b - a > 1) {
                    const uint32_t c = a + (b - a) / 2;
                    if (slot_of(c) == k) a = c; else b = c;
                }
            }
            const uint32_t b_hi = a;
            const float x_small = sg ? value(b_hi) : value(b_lo);
            const float x_large = sg ? value(b_lo) : value(b_hi);
            const uint32_t c0 = count_below(smid, x_small);
            const uint32_t c1 = count_below(smid, x_large);
            if (k >= count) {
                why = "a quotient converts to a half float outside the slot table";
                return false;
            }
            if (c1 < c0 || c1 - c0 > 1) {
                why = "a lookup slot spans more than one quantisation midpoint";
                return false;
            }
            eri::KeySlot s;
            s.lo = c0;
            s.mid = (c1 == c0) ? inf : smid[c0];
            std::memcpy(out + (size_t)k * stride, &s, sizeof s);
            b_lo = b_hi + 1;
        }
    }
    return true;
}

const Tables &tables() {
    static Tables t;
    static std::once_flag once;
    std::call_once(once, [] {
        for (int i = 0; i < 256; ++i) {
            t.map_s[i] = bits_to_float(ERI_DYNAMIC_MAP_SIGNED_BITS[i]);
            t.map_u[i] = bits_to_float(ERI_DYNAMIC_MAP_UNSIGNED_BITS[i]);
        }
        for (int j = 0; j < 255; ++j) {
            float s = t.map_s[j] + t.map_s[j + 1];
            t.mid_s[j] = s * 0.5f;
            float u = t.map_u[j] + t.map_u[j + 1];
            t.mid_u[j] = u * 0.5f;
        }
        t.mid_s[255] = t.mid_u[255] = std::numeric_limits<float>::infinity();
        for (int j = 0; j < 255; ++j) {
            if (!(t.map_s[j] < t.map_s[j + 1]) || !(t.map_u[j] < t.map_u[j + 1])) {
                t.why = "quantisation map is not strictly increasing";
                return;
            }
        }
        if (t.map_s[127] != 0.0f || t.map_u[0] != 0.0f || t.map_s[255] != 1.0f || t.map_u[255] != 1.0f) {
            t.why = "quantisation map lost its fixed points";
            return;
        }
        t.image.assign(eri::kLdsImageBytes, 0);
        std::memcpy(&t.image[eri::kOffMapS], t.map_s, 1024);
        std::memcpy(&t.image[eri::kOffMapU], t.map_u, 1024);
        std::memcpy(&t.image[eri::kOffMidS], t.mid_s, 1024);
        std::memcpy(&t.image[eri::kOffMidU], t.mid_u, 1024);
        if (!build_slots(t.mid_s, eri::kSKeyDrop, 0xffffu, eri::kSKeyStride, eri::kSKeyCount, &t.image[eri::kOffKeyS], t.why)) return;
        if (!build_slots(t.mid_u, eri::kUKeyDrop, 0x7fffu, eri::kUKeyStride, eri::kUKeyCount, &t.image[eri::kOffKeyU], t.why)) return;
        t.ok = true;
    });
    return t;
}

// ---------------------------------------------------------------------------------------------
// per-device context
// ---------------------------------------------------------------------------------------------

constexpr int kMaxDevices = 16;

/* Scratch of eri_adam8_grad_norm_static: the per-wave partial sums of the gradient-norm pass, in device
 * memory that exists from the moment the library is loaded until the process ends (every device the
 * library runs on holds its own copy, 384 KiB).  The name below is a host-side stand-in, not a device
 * address: host code uses DeviceCtx::scratch_ptr, which hipGetSymbolAddress filled in for that device. */
constexpr uint32_t kNormScratchPairs = 24576; // {sum of squares, non-finite count} per wave: 3 groups x 256 CUs x 32 waves
static __device__ __align__(256) double scratch[2 * kNormScratchPairs];

struct DeviceCtx {
    void *image = nullptr; // device copy of the LDS image
    double *scratch_ptr = nullptr; // address of this device's copy of the static array `scratch`
    uint32_t cus = 0;
    uint32_t wg = 1024;      // threads per workgroup: the table image (~100 KB of LDS) allows one per CU
    uint32_t wg_per_cu = 1;  // persistent workgroups per compute unit
    bool ready = false;
};

DeviceCtx g_ctx[kMaxDevices];
std::mutex g_ctx_mu;

int get_ctx(DeviceCtx **out) {
    int dev = 0;
    ERI_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(ERI_ERR_ARG, "device index out of range");
    std::lock_guard<std::mutex> lk(g_ctx_mu);
    DeviceCtx &c = g_ctx[dev];
    if (!c.ready) {
        const Tables &t = tables();
        if (!t.ok) return fail(ERI_ERR_INTERNAL, "quantisation tables failed their self-check: " + t.why);
        hipDeviceProp_t prop;
        ERI_HIP(hipGetDeviceProperties(&prop, dev));
        c.cus = (uint32_t)prop.multiProcessorCount;
        void *image = nullptr;
        ERI_HIP(hipMalloc(&image, eri::kLdsImageBytes));
        const hipError_t e = hipMemcpy(image, t.image.data(), eri::kLdsImageBytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(image);
            return hip_fail(e, "upload of the quantisation tables");
        }
        double *ptr = nullptr; // once per device, with that device current
        const hipError_t se = hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch));
        if (se != hipSuccess || !ptr) {
            (void)hipFree(image);
            return hip_fail(se != hipSuccess ? se : hipErrorInvalidSymbol, "address of the static gradient-norm scratch");
        }
        c.scratch_ptr = ptr;
        c.image = image;
        c.ready = true;
    }
    *out = &c;
    return 0;
}

/* The context of the current device, which must be the one the table was created on: its rows and
 * the table image are addresses of that device. */
int get_ctx_on(int table_device, DeviceCtx **out) {
    int rc = get_ctx(out);
    if (rc) return rc;
    if (*out != &g_ctx[table_device]) {
        int dev = 0;
        (void)hipGetDevice(&dev);
        char buf[96];
        std::snprintf(buf, sizeof buf, "table belongs to device %d, current device is %d", table_device, dev);
        return fail(ERI_ERR_ARG, buf);
    }
    return 0;
}

constexpr size_t kRecycleThreshold = (size_t)64 << 20;

bool recycle_enabled() {
    static const bool on = [] {
        const char *s = std::getenv("ERI_HIP_MALLOC_RECYCLE");
        return !(s && s[0] == '0');
    }();
    return on;
}

uint64_t blocks_of(uint64_t numel) { return (numel + eri::kBlock - 1) / eri::kBlock; }

} // namespace

// ---------------------------------------------------------------------------------------------
// launch table
// ---------------------------------------------------------------------------------------------

struct EriAdam8Table {
    struct Group {
        int dtype = 0;
        uint32_t n = 0;
        uint32_t total_blocks = 0; // full blocks only; a row's partial last block is handled per row
        eri::DevTensor *dev = nullptr;    // n rows, then one uint32 row index per full block (BlockRowMap)
        eri::DevTensor *pinned = nullptr; // the rows only
        std::vector<uint32_t> src; // index into the caller's rows
        bool unit_scales = true;   // every row's grad_scale is exactly 1
    };
    int device = 0;
    uint32_t n = 0;
    uint64_t total_numel = 0;
    uint64_t total_blocks = 0;
    Group groups[eri::kLayouts]; // F32, BF16, BF16 with F32 gradients
    std::vector<uint64_t> numel;
    std::vector<int32_t> dtype; // per row: its layout
    hipEvent_t uploaded = nullptr;
    bool upload_pending = false;
    void *upload_stream = nullptr;  // stream of the last upload
    void *ordered_stream = nullptr; // another stream that has already been made to wait for that upload
    bool ordered_valid = false;
    double *partial = nullptr; // one sum of squares per wave of the norm pass, per group
    float *norm_out = nullptr; // device: {norm, clip factor, 64-bit count}, owned by the table
    float *norm_last = nullptr; // where the last norm pass left its result: norm_out, the caller's buffer, or the
                                // norm_out of the table this one was normed together with
    bool grads_only = false;    // rows carry gradients only: the table serves the norm pass and nothing else
    uint32_t n_partial = 0;
    double *qerr = nullptr;    // device: per row {sum |m - deq m|, sum |v - deq v|}, groups back to back
    bool qerr_valid = false;
};

namespace {

int layout_of(const EriAdam8Tensor &r) {
    if (r.dtype_tag == ERI_DTYPE_F32) return eri::kLayoutF32;
    return r.grad_f32 ? eri::kLayoutBF16GradF32 : eri::kLayoutBF16;
}

int validate_rows(const EriAdam8Tensor *rows, uint32_t n, bool grads_only = false) {
    if (!rows) return fail(ERI_ERR_NULL, "rows is NULL");
    if (n == 0) return fail(ERI_ERR_ARG, "launch table has no rows");
    uint64_t running = 0;
    char buf[160];
    for (uint32_t i = 0; i < n; ++i) {
        const EriAdam8Tensor &r = rows[i];
        if (grads_only ? !r.g : (!r.p || !r.g || !r.m || !r.v || !r.absmax_m || !r.absmax_v)) {
            std::snprintf(buf, sizeof buf, "row %u: NULL pointer", i);
            return fail(ERI_ERR_NULL, buf);
        }
        if (r.numel == 0) {
            std::snprintf(buf, sizeof buf, "row %u: Empty tensor for quantization", i);
            return fail(ERI_ERR_EMPTY, buf);
        }
        if (r.dtype_tag != ERI_DTYPE_F32 && r.dtype_tag != ERI_DTYPE_BF16) {
            std::snprintf(buf, sizeof buf, "row %u: unsupported dtype tag %d (F32=0 and BF16=2 are supported)", i,
                          r.dtype_tag);
            return fail(ERI_ERR_DTYPE, buf);
        }
        if (r.grad_f32 && r.dtype_tag == ERI_DTYPE_F32) {
            std::snprintf(buf, sizeof buf, "row %u: grad_f32 is for BF16 parameters (F32 parameters take F32 gradients anyway)", i);
            return fail(ERI_ERR_DTYPE, buf);
        }
        if (r.p_src && r.p_src != r.p) {
            const uintptr_t bytes = (uintptr_t)r.numel * (r.dtype_tag == ERI_DTYPE_F32 ? 4u : 2u);
            const uintptr_t a = (uintptr_t)r.p, b = (uintptr_t)r.p_src;
            if (a < b + bytes && b < a + bytes) {
                std::snprintf(buf, sizeof buf, "row %u: p_src overlaps p without being equal to it", i);
                return fail(ERI_ERR_ARG, buf);
            }
        }
        const uintptr_t wide = (uintptr_t)r.p | (uintptr_t)r.g | (uintptr_t)r.m | (uintptr_t)r.v | (uintptr_t)r.p_src |
                               (uintptr_t)r.ema_shadow;
        const uintptr_t narrow = (uintptr_t)r.absmax_m | (uintptr_t)r.absmax_v;
        if ((wide & 15u) || (narrow & 3u)) {
            std::snprintf(buf, sizeof buf, "row %u: p/g/m/v must be 16-byte aligned, absmax 4-byte aligned", i);
            return fail(ERI_ERR_ALIGN, buf);
        }
        if (r.block_start != running) {
            std::snprintf(buf, sizeof buf, "row %u: block_start %llu, expected %llu", i,
                          (unsigned long long)r.block_start, (unsigned long long)running);
            return fail(ERI_ERR_BLOCK_START, buf);
        }
        running += blocks_of(r.numel);
    }
    if (running > 0x7fffffffull) return fail(ERI_ERR_TOO_LARGE, "more than 2^31 - 1 blocks in one table");
    return 0;
}

void fill_group(EriAdam8Table::Group &g, const EriAdam8Tensor *rows) {
    uint32_t start = 0;
    g.unit_scales = true;
    for (uint32_t j = 0; j < g.n; ++j) {
        if (rows[g.src[j]].grad_scale != 1.0f) g.unit_scales = false;
        const EriAdam8Tensor &r = rows[g.src[j]];
        eri::DevTensor &d = g.pinned[j];
        d.p = r.p;
        d.p_in = r.p_src ? r.p_src : r.p;
        d.shadow = r.ema_shadow;
        d.g = r.g;
        d.m = r.m;
        d.v = r.v;
        d.absmax_m = r.absmax_m;
        d.absmax_v = r.absmax_v;
        d.numel = r.numel;
        d.full_start = start;
        d.grad_scale = r.grad_scale;
        start += (uint32_t)(r.numel / eri::kBlock);
    }
    g.total_blocks = start;
}

int upload(EriAdam8Table *t, void *stream) {
    for (auto &g : t->groups) {
        if (g.n == 0) continue;
        ERI_HIP(hipMemcpyAsync(g.dev, g.pinned, sizeof(eri::DevTensor) * g.n, hipMemcpyHostToDevice,
                               static_cast<hipStream_t>(stream)));
    }
    ERI_HIP(hipEventRecord(t->uploaded, static_cast<hipStream_t>(stream)));
    t->upload_pending = true;
    t->upload_stream = stream;
    t->ordered_valid = false;
    return 0;
}

/* Work that reads the device rows must run after their upload.  On the upload's own stream that is stream
 * order; another stream is made to wait for the upload's event (no host wait).  A stream that is being
 * captured into a graph cannot wait for an event outside the graph, so there the host waits for the
 * upload instead, once. */
int order_after_upload(EriAdam8Table *t, void *stream) {
    if (!t->upload_pending || stream == t->upload_stream) return 0;
    if (t->ordered_valid && stream == t->ordered_stream) return 0;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &cs) != hipSuccess) {
        (void)hipGetLastError();
        cs = hipStreamCaptureStatusNone;
    }
    if (cs == hipStreamCaptureStatusActive) {
        const hipError_t e = hipEventSynchronize(t->uploaded);
        if (e != hipSuccess) {
            hip_fail(e, "hipEventSynchronize");
            return fail((int)e, "the launch table was uploaded on another stream and that copy may not have finished: "
                                "create or update the table on the stream being captured, or synchronise before the capture");
        }
        t->upload_pending = false;
        return 0;
    }
    ERI_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), t->uploaded, 0));
    t->ordered_stream = stream;
    t->ordered_valid = true;
    return 0;
}

void destroy_table(EriAdam8Table *t) {
    if (!t) return;
    for (auto &g : t->groups) {
        if (g.dev) (void)hipFree(g.dev);
        if (g.pinned) (void)hipHostFree(g.pinned);
    }
    if (t->uploaded) (void)hipEventDestroy(t->uploaded);
    if (t->partial) (void)hipFree(t->partial);
    if (t->norm_out) (void)hipFree(t->norm_out);
    if (t->qerr) (void)hipFree(t->qerr);
    delete t;
}

} // namespace

extern "C" {

const char *eri_last_error(void) { return g_err.c_str(); }

void eri_set_last_error(const char *message) { g_err = message ? message : ""; }

// ---- storage --------------------------------------------------------------------------------

int eri_hip_device_count(int *count) {
    if (!count) return fail(ERI_ERR_NULL, "count is NULL");
    ERI_HIP(hipGetDeviceCount(count));
    return 0;
}

int eri_hip_set_device(int device) {
    ERI_HIP(hipSetDevice(device));
    return 0;
}

int eri_hip_get_device(int *device) {
    if (!device) return fail(ERI_ERR_NULL, "device is NULL");
    ERI_HIP(hipGetDevice(device));
    return 0;
}

int eri_hip_malloc_zeroed(int device, size_t bytes, void **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (bytes == 0) return fail(ERI_ERR_ARG, "zero-byte allocation");
    int prev = 0;
    ERI_HIP(hipGetDevice(&prev));
    if (prev != device) ERI_HIP(hipSetDevice(device));
    void *p = nullptr;
    auto device_alloc = [&](void **q) -> hipError_t { return hipMalloc(q, bytes); };
    hipError_t e = device_alloc(&p);
    // Placement conditioning.  On MI355X the first physical placement a large allocation receives
    // sustains visibly less write bandwidth than the placement the same request receives once the
    // range has been handed back to the driver (measured with a plain streaming kernel: 4.6 vs
    // 5.5 TB/s on 24 GB buffers).  Large allocations are therefore allocated, released and
    // allocated again.  ERI_HIP_MALLOC_RECYCLE=0 switches this off.
    if (e == hipSuccess && bytes >= kRecycleThreshold && recycle_enabled()) {
        e = hipFree(p);
        p = nullptr;
        if (e == hipSuccess) e = device_alloc(&p);
    }
    if (e == hipSuccess) e = hipMemset(p, 0, bytes);
    if (prev != device) (void)hipSetDevice(prev);
    if (e != hipSuccess) {
        if (p) (void)hipFree(p);
        return hip_fail(e, "hipMalloc/hipMemset");
    }
    *out = p;
    return 0;
}

int eri_hip_free(void *ptr) {
    if (!ptr) return 0;
    ERI_HIP(hipFree(ptr));
    return 0;
}

} // extern "C"

struct EriHipPool {
    int device = 0;
    char *base = nullptr;
    size_t lane_bytes = 0;
    std::vector<size_t> used; // per lane: bytes handed out from the lane's start upwards
    struct Piece {
        size_t offset, bytes; // inside the lane
    };
    std::vector<std::vector<Piece>> released; // per lane: pieces given back below the lane's top
    std::mutex lock;
    int refs = 1;        // the creator's reference plus one per eri_hip_pool_retain (guarded by lock)
    bool closed = false; // the creator has let go: nothing more is handed out
};

namespace {

/* Takes `need` bytes (a multiple of 256) out of `lane`: a released piece of exactly that size if there is one,
 * else the next bytes above the lane's top. */
char *pool_take(EriHipPool *pool, uint32_t lane, size_t need) {
    auto &back = pool->released[lane];
    for (size_t i = 0; i < back.size(); ++i) {
        if (back[i].bytes == need) {
            char *p = pool->base + (size_t)lane * pool->lane_bytes + back[i].offset;
            back[i] = back.back();
            back.pop_back();
            return p;
        }
    }
    if (need > pool->lane_bytes - pool->used[lane]) return nullptr;
    char *p = pool->base + (size_t)lane * pool->lane_bytes + pool->used[lane];
    pool->used[lane] += need;
    return p;
}

} // namespace

extern "C" {

int eri_hip_pool_create(int device, size_t bytes, uint32_t lanes, EriHipPool **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    int prev = 0;
    ERI_HIP(hipGetDevice(&prev));
    if (prev != device) ERI_HIP(hipSetDevice(device));
    hipError_t e = hipSuccess;
    if (bytes == 0) {
        size_t free_b = 0, total_b = 0;
        e = hipMemGetInfo(&free_b, &total_b);
        bytes = free_b / 10 * 9;
    }
    constexpr size_t kGrain = (size_t)2 << 20;       // lanes start on 2 MiB boundaries
    constexpr size_t kDefaultLane = (size_t)48 << 30; // the distance at which the step ran fastest
    size_t lane_bytes;
    if (lanes == 0) { // as many 48 GiB lanes as fit; a smaller pool is one lane
        lanes = (uint32_t)(bytes / kDefaultLane);
        lane_bytes = lanes ? kDefaultLane : bytes / kGrain * kGrain;
        if (lanes == 0) lanes = 1;
    } else {
        lane_bytes = bytes / lanes / kGrain * kGrain;
    }
    void *p = nullptr;
    if (e == hipSuccess && lane_bytes == 0) e = hipErrorInvalidValue;
    if (e == hipSuccess) e = hipMalloc(&p, lane_bytes * lanes);
    if (prev != device) (void)hipSetDevice(prev);
    if (e != hipSuccess) return hip_fail(e, "memory pool allocation");
    EriHipPool *pool = new EriHipPool();
    pool->device = device;
    pool->base = static_cast<char *>(p);
    pool->lane_bytes = lane_bytes;
    pool->used.assign(lanes, 0);
    pool->released.assign(lanes, {});
    *out = pool;
    return 0;
}

int eri_hip_pool_alloc_zeroed(EriHipPool *pool, uint32_t lane, size_t bytes, void **out) {
    if (!pool || !out) return fail(ERI_ERR_NULL, "pool or out is NULL");
    *out = nullptr;
    if (bytes == 0) return fail(ERI_ERR_EMPTY, "pool allocation of zero bytes");
    const size_t need = (bytes + 255) / 256 * 256;
    char *p = nullptr;
    {
        std::lock_guard<std::mutex> g(pool->lock);
        if (pool->closed) return fail(ERI_ERR_ARG, "memory pool: the pool has been destroyed");
        p = pool_take(pool, lane % (uint32_t)pool->used.size(), need);
    }
    if (!p) return fail(ERI_ERR_ARG, "memory pool: the lane is full");
    int prev = 0;
    ERI_HIP(hipGetDevice(&prev));
    if (prev != pool->device) ERI_HIP(hipSetDevice(pool->device));
    const hipError_t e = hipMemset(p, 0, bytes);
    if (prev != pool->device) (void)hipSetDevice(prev);
    if (e != hipSuccess) {
        (void)eri_hip_pool_release(pool, p, bytes);
        return hip_fail(e, "hipMemset");
    }
    *out = p;
    return 0;
}

int eri_hip_pool_alloc_zeroed_async(EriHipPool *pool, uint32_t lane, size_t bytes, void *stream, void **out) {
    if (!pool || !out) return fail(ERI_ERR_NULL, "pool or out is NULL");
    *out = nullptr;
    if (bytes == 0) return fail(ERI_ERR_EMPTY, "pool allocation of zero bytes");
    const size_t need = (bytes + 255) / 256 * 256;
    char *p = nullptr;
    {
        std::lock_guard<std::mutex> g(pool->lock);
        if (pool->closed) return fail(ERI_ERR_ARG, "memory pool: the pool has been destroyed");
        p = pool_take(pool, lane % (uint32_t)pool->used.size(), need);
    }
    if (!p) return fail(ERI_ERR_ARG, "memory pool: the lane is full");
    int prev = 0;
    ERI_HIP(hipGetDevice(&prev));
    if (prev != pool->device) ERI_HIP(hipSetDevice(pool->device));
    // pieces are 256-byte aligned and so is `need`: the whole piece is cleared, with a kernel (a memset node in
    // a captured graph is not reliable on this stack, and the runtime's synchronous memset blocks the host)
    const int rc = eri::launch_fill_zero(p, need, stream);
    if (prev != pool->device) (void)hipSetDevice(prev);
    if (rc) {
        (void)eri_hip_pool_release(pool, p, bytes);
        return hip_fail((hipError_t)rc, "fill kernel");
    }
    *out = p;
    return 0;
}

int eri_hip_pool_release(EriHipPool *pool, void *ptr, size_t bytes) {
    if (!pool) return fail(ERI_ERR_NULL, "pool is NULL");
    if (!ptr) return 0;
    const size_t need = (bytes + 255) / 256 * 256;
    char *p = static_cast<char *>(ptr);
    std::lock_guard<std::mutex> g(pool->lock);
    const size_t lanes = pool->used.size();
    if (bytes == 0 || p < pool->base || p >= pool->base + pool->lane_bytes * lanes)
        return fail(ERI_ERR_ARG, "memory pool: release of a piece that is not the pool's");
    const size_t lane = (size_t)(p - pool->base) / pool->lane_bytes;
    const size_t offset = (size_t)(p - pool->base) % pool->lane_bytes;
    if (offset % 256 != 0 || offset + need > pool->used[lane])
        return fail(ERI_ERR_ARG, "memory pool: release of a piece that is not the pool's");
    for (const auto &piece : pool->released[lane]) // a second release would hand the same bytes out twice
        if (offset < piece.offset + piece.bytes && piece.offset < offset + need)
            return fail(ERI_ERR_ARG, "memory pool: the piece, or a part of it, has been released already");
    if (offset + need == pool->used[lane]) { // the top piece: the lane shrinks, and so it does past released pieces below it
        pool->used[lane] = offset;
        auto &back = pool->released[lane];
        for (bool again = true; again;) {
            again = false;
            for (size_t i = 0; i < back.size(); ++i) {
                if (back[i].offset + back[i].bytes == pool->used[lane]) {
                    pool->used[lane] = back[i].offset;
                    back[i] = back.back();
                    back.pop_back();
                    again = true;
                    break;
                }
            }
        }
    } else {
        pool->released[lane].push_back({offset, need});
    }
    return 0;
}

int eri_hip_pool_info(const EriHipPool *pool, uint32_t *lanes, size_t *lane_bytes) {
    if (!pool) return fail(ERI_ERR_NULL, "pool is NULL");
    if (lanes) *lanes = (uint32_t)pool->used.size();
    if (lane_bytes) *lane_bytes = pool->lane_bytes;
    return 0;
}

int eri_hip_pool_lane_used(const EriHipPool *pool, uint32_t lane, size_t *used_bytes) {
    if (!pool || !used_bytes) return fail(ERI_ERR_NULL, "pool or used_bytes is NULL");
    std::lock_guard<std::mutex> g(const_cast<EriHipPool *>(pool)->lock);
    *used_bytes = pool->used[lane % pool->used.size()];
    return 0;
}

int eri_hip_pool_reset(EriHipPool *pool) {
    if (!pool) return fail(ERI_ERR_NULL, "pool is NULL");
    std::lock_guard<std::mutex> g(pool->lock);
    for (auto &u : pool->used) u = 0;
    for (auto &r : pool->released) r.clear();
    return 0;
}

int eri_hip_pool_retain(EriHipPool *pool) {
    if (!pool) return fail(ERI_ERR_NULL, "pool is NULL");
    std::lock_guard<std::mutex> g(pool->lock);
    pool->refs += 1;
    return 0;
}

static int pool_unref(EriHipPool *pool, bool creator) {
    bool last;
    {
        std::lock_guard<std::mutex> g(pool->lock);
        if (creator) pool->closed = true;
        pool->refs -= 1;
        last = pool->refs <= 0;
    }
    if (!last) return 0;
    const hipError_t e = hipFree(pool->base);
    delete pool;
    if (e != hipSuccess) return hip_fail(e, "hipFree");
    return 0;
}

int eri_hip_pool_destroy(EriHipPool *pool) {
    if (!pool) return 0;
    return pool_unref(pool, true);
}

int eri_hip_pool_unretain(EriHipPool *pool) {
    if (!pool) return 0;
    return pool_unref(pool, false);
}

void *eri_hip_host_alloc(size_t bytes) {
    void *p = nullptr;
    hipError_t e = hipHostMalloc(&p, bytes, hipHostMallocPortable);
    if (e != hipSuccess) {
        hip_fail(e, "hipHostMalloc");
        return nullptr;
    }
    return p;
}

int eri_hip_host_free(void *ptr) {
    if (!ptr) return 0;
    ERI_HIP(hipHostFree(ptr));
    return 0;
}

int eri_hip_memcpy_async(void *dst, const void *src, size_t bytes, int kind, void *stream) {
    if (bytes == 0) return 0;
    if (!dst || !src) return fail(ERI_ERR_NULL, "memcpy with NULL pointer");
    hipMemcpyKind k = hipMemcpyDefault;
    if (kind == 1) k = hipMemcpyHostToDevice;
    else if (kind == 2) k = hipMemcpyDeviceToHost;
    else if (kind == 3) k = hipMemcpyDeviceToDevice;
    ERI_HIP(hipMemcpyAsync(dst, src, bytes, k, static_cast<hipStream_t>(stream)));
    return 0;
}

int eri_hip_memset_async(void *dst, int value, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    if (!dst) return fail(ERI_ERR_NULL, "memset with NULL pointer");
    ERI_HIP(hipMemsetAsync(dst, value, bytes, static_cast<hipStream_t>(stream)));
    return 0;
}

int eri_hip_stream_create(void **stream) {
    if (!stream) return fail(ERI_ERR_NULL, "stream is NULL");
    hipStream_t s = nullptr;
    ERI_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return 0;
}

int eri_hip_stream_sync(void *stream) {
    ERI_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return 0;
}

int eri_hip_stream_destroy(void *stream) {
    if (!stream) return 0;
    ERI_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return 0;
}

int eri_hip_mem_info(size_t *free_bytes, size_t *total_bytes) {
    size_t f = 0, t = 0;
    ERI_HIP(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

int eri_hip_pointer_kind(const void *p, int *kind) {
    if (!kind) return fail(ERI_ERR_NULL, "kind is NULL");
    *kind = ERI_PTR_UNKNOWN;
    if (!p) return 0;
    hipPointerAttribute_t a;
    std::memset(&a, 0, sizeof a);
    const hipError_t e = hipPointerGetAttributes(&a, p);
    if (e == hipErrorInvalidValue) { // how older runtimes answer for memory they did not allocate
        (void)hipGetLastError();
        return 0;
    }
    if (e != hipSuccess) return hip_fail(e, "hipPointerGetAttributes");
    switch (a.type) {
    case hipMemoryTypeDevice: case hipMemoryTypeArray: *kind = ERI_PTR_DEVICE; break;
    case hipMemoryTypeHost: *kind = ERI_PTR_PINNED_HOST; break;
    case hipMemoryTypeManaged: case hipMemoryTypeUnified: *kind = ERI_PTR_MANAGED; break;
    default: *kind = ERI_PTR_UNKNOWN; break;
    }
    return 0;
}

/* The checkpoint calls below run a kernel on pointers that come straight from a caller who is often handling
 * host buffers at that moment; ordinary host memory handed to a kernel is a memory fault of the whole device,
 * so these calls (none of them is on a step's path) ask the runtime first. */
static int require_kernel_visible(const void *p, const char *what) {
    int kind = ERI_PTR_UNKNOWN;
    const int rc = eri_hip_pointer_kind(p, &kind);
    if (rc) return rc;
    if (kind == ERI_PTR_UNKNOWN)
        return fail(ERI_ERR_ARG, std::string(what) + " is not device, pinned or managed memory: kernels cannot reach it");
    return 0;
}

// ---- optimizer ------------------------------------------------------------------------------

int eri_adam8_init(void) {
    DeviceCtx *c = nullptr;
    return get_ctx(&c);
}

int eri_adam8_get_maps(float *signed256, float *unsigned256) {
    const Tables &t = tables();
    if (!t.ok) return fail(ERI_ERR_INTERNAL, "quantisation tables failed their self-check: " + t.why);
    if (signed256) std::memcpy(signed256, t.map_s, 1024);
    if (unsigned256) std::memcpy(unsigned256, t.map_u, 1024);
    return 0;
}

int eri_adam8_table_image(void *out, size_t cap, size_t *bytes, uint32_t offsets[6]) {
    const Tables &t = tables();
    if (!t.ok) return fail(ERI_ERR_INTERNAL, "quantisation tables failed their self-check: " + t.why);
    if (bytes) *bytes = t.image.size();
    if (offsets) {
        const uint32_t o[6] = {eri::kOffMapS, eri::kOffMapU, eri::kOffMidS, eri::kOffMidU, eri::kOffKeyS, eri::kOffKeyU};
        std::memcpy(offsets, o, sizeof o);
    }
    if (out) {
        if (cap < t.image.size()) return fail(ERI_ERR_ARG, "table image does not fit the buffer");
        std::memcpy(out, t.image.data(), t.image.size());
    }
    return 0;
}

int eri_adam8_hyper_pack(double lr, double beta1, double beta2, double eps, double weight_decay, uint64_t step,
                         int mode, uint32_t flags, EriAdam8Hyper *out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    if (mode != ERI_ADAM8_MODE_ERI && mode != ERI_ADAM8_MODE_L2 && mode != ERI_ADAM8_MODE_BNB)
        return fail(ERI_ERR_ARG, "unknown mode");
    std::memset(out, 0, sizeof(*out));
    out->mode = mode;
    out->flags = flags;
    out->beta1 = (float)beta1;
    out->beta2 = (float)beta2;
    out->eps = (float)eps;
    out->weight_decay = (float)weight_decay;
    out->grad_scale = 1.0f;
    if (mode == ERI_ADAM8_MODE_L2) {
        const uint64_t s = step < 1 ? 1 : step;               // adam8bit.rs:164
        out->omb1 = (float)(1.0 - beta1);                      // :142  f64 subtraction, then the cast
        out->omb2 = (float)(1.0 - beta2);                      // :151
        out->bc1 = (float)(1.0 - std::pow(beta1, (double)(int32_t)s)); // :167 powi
        out->bc2 = (float)(1.0 - std::pow(beta2, (double)(int32_t)s)); // :175
        out->step_size = (float)lr;                            // :193
    } else {
        const double t = (double)step;                         // adam8bit_enhanced.rs:210
        const double bc1 = 1.0 - std::pow(beta1, t);           // :213
        const double bc2 = 1.0 - std::pow(beta2, t);           // :214
        out->omb1 = 1.0f - out->beta1;                         // :256  `1.0 - beta1 as f32`
        out->omb2 = 1.0f - out->beta2;                         // :260
        out->bc1 = (float)bc1;
        out->bc2 = (float)bc2;
        out->step_size = (float)(lr * (std::sqrt(bc2) / bc1)); // :215, cast at :274
        if (mode == ERI_ADAM8_MODE_BNB) {
            out->eps = (float)(eps * std::sqrt(bc2));
            out->weight_decay = (float)(1.0 - lr * weight_decay); // decay factor
        }
    }
    return 0;
}

int eri_adam8_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel, void *stream) {
    if (!m || !v || !absmax_m || !absmax_v) return fail(ERI_ERR_NULL, "state pointer is NULL");
    if (numel == 0) return fail(ERI_ERR_EMPTY, "Empty tensor for quantization");
    int rc = eri::launch_state_init(m, v, absmax_m, absmax_v, numel, stream);
    if (rc) return hip_fail((hipError_t)rc, "state_init launch");
    return 0;
}

static int table_create(const EriAdam8Tensor *rows, uint32_t n, bool grads_only, void *stream, EriAdam8Table **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    int rc = validate_rows(rows, n, grads_only);
    if (rc) return rc;
    DeviceCtx *ctx = nullptr;
    rc = get_ctx(&ctx);
    if (rc) return rc;
    EriAdam8Table *t = new EriAdam8Table();
    t->n = n;
    t->grads_only = grads_only;
    (void)hipGetDevice(&t->device);
    for (int li = 0; li < eri::kLayouts; ++li) t->groups[li].dtype = li; // a Layout
    t->numel.resize(n);
    t->dtype.resize(n);
    for (uint32_t i = 0; i < n; ++i) {
        t->numel[i] = rows[i].numel;
        t->dtype[i] = layout_of(rows[i]);
        t->total_numel += rows[i].numel;
        t->total_blocks += blocks_of(rows[i].numel);
        t->groups[layout_of(rows[i])].src.push_back(i);
    }
    hipError_t e = hipEventCreateWithFlags(&t->uploaded, hipEventDisableTiming);
    for (auto &g : t->groups) {
        g.n = (uint32_t)g.src.size();
        if (g.n == 0 || e != hipSuccess) continue;
        uint64_t full = 0;
        for (uint32_t j = 0; j < g.n; ++j) full += rows[g.src[j]].numel / eri::kBlock;
        e = hipMalloc((void **)&g.dev, sizeof(eri::DevTensor) * g.n + sizeof(uint32_t) * (full ? full : 1));
        if (e == hipSuccess) e = hipHostMalloc((void **)&g.pinned, sizeof(eri::DevTensor) * g.n, hipHostMallocDefault);
        if (e == hipSuccess) fill_group(g, rows);
        if (e == hipSuccess && full) { // which row owns which full block: fixed for the table's life
            std::vector<uint32_t> row_of((size_t)full);
            size_t at = 0;
            for (uint32_t j = 0; j < g.n; ++j)
                for (uint64_t k = rows[g.src[j]].numel / eri::kBlock; k > 0; --k) row_of[at++] = j;
            e = hipMemcpy(g.dev + g.n, row_of.data(), sizeof(uint32_t) * (size_t)full, hipMemcpyHostToDevice);
        }
    }
    if (e != hipSuccess) {
        destroy_table(t);
        return hip_fail(e, "launch table allocation");
    }
    rc = upload(t, stream);
    if (rc) {
        destroy_table(t);
        return rc;
    }
    *out = t;
    return 0;
}

int eri_adam8_table_create(const EriAdam8Tensor *rows, uint32_t n, void *stream, EriAdam8Table **out) {
    return table_create(rows, n, false, stream, out);
}

int eri_adam8_grad_table_create(const EriAdam8Tensor *rows, uint32_t n, void *stream, EriAdam8Table **out) {
    return table_create(rows, n, true, stream, out);
}

int eri_adam8_table_update(EriAdam8Table *t, const EriAdam8Tensor *rows, uint32_t n, void *stream) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    int rc = validate_rows(rows, n, t->grads_only);
    if (rc) return rc;
    if (n != t->n) return fail(ERI_ERR_ARG, "table_update: row count differs from the table's");
    for (uint32_t i = 0; i < n; ++i)
        if (rows[i].numel != t->numel[i] || layout_of(rows[i]) != t->dtype[i])
            return fail(ERI_ERR_ARG, "table_update: numel or dtype differs from the table's");
    if (t->upload_pending) { // the pinned mirror may still be the source of the previous copy
        ERI_HIP(hipEventSynchronize(t->uploaded));
        t->upload_pending = false;
    }
    for (auto &g : t->groups)
        if (g.n) fill_group(g, rows);
    return upload(t, stream);
}

int eri_adam8_table_destroy(EriAdam8Table *t) {
    destroy_table(t);
    return 0;
}

int eri_adam8_table_info(const EriAdam8Table *t, uint64_t *total_numel, uint64_t *total_blocks) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    if (total_numel) *total_numel = t->total_numel;
    if (total_blocks) *total_blocks = t->total_blocks;
    return 0;
}

int eri_adam8_step_table(EriAdam8Table *t, const EriAdam8Hyper *h, void *stream) {
    if (!t || !h) return fail(ERI_ERR_NULL, "table or hyper is NULL");
    if (t->grads_only) return fail(ERI_ERR_ARG, "a gradient-only table serves eri_adam8_grad_norm only");
    if (h->mode != ERI_ADAM8_MODE_ERI && h->mode != ERI_ADAM8_MODE_L2 && h->mode != ERI_ADAM8_MODE_BNB)
        return fail(ERI_ERR_ARG, "unknown mode");
    if ((h->flags & ERI_ADAM8_FLAG_EMA) && !(h->ema_decay >= 0.0f && h->ema_decay <= 1.0f))
        return fail(ERI_ERR_ARG, "ERI_ADAM8_FLAG_EMA needs ema_decay in [0, 1]");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx_on(t->device, &ctx);
    if (rc) return rc;
    const bool clip = (h->flags & ERI_ADAM8_FLAG_CLIP_FROM_TABLE) != 0;
    const bool scaled = (h->flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
    if (clip) { // checked for every group before the first launch: a refused step changes nothing
        if (!t->norm_last) return fail(ERI_ERR_ARG, "ERI_ADAM8_FLAG_CLIP_FROM_TABLE without a prior eri_adam8_grad_norm");
        for (auto &g : t->groups)
            if (g.n && !scaled && !g.unit_scales)
                return fail(ERI_ERR_ARG, "ERI_ADAM8_FLAG_CLIP_FROM_TABLE needs per-tensor grad_scale = 1 unless ERI_ADAM8_FLAG_GRAD_SCALE is set");
    }
    rc = order_after_upload(t, stream);
    if (rc) return rc;
    std::vector<EriEmaTensor> ema_rest;
    for (auto &g : t->groups) {
        if (g.n == 0) continue;
        // One wavefront per block.  A small table gets smaller workgroups so that its blocks still
        // spread over every compute unit instead of filling a few of them.
        uint32_t waves_per_wg = ctx->wg / eri::kWave;
        const uint32_t slots = ctx->cus * ctx->wg_per_cu;
        const uint32_t work = g.total_blocks > g.n ? g.total_blocks : g.n; // full blocks, or one tail per row
        const uint32_t per_slot = (work + slots - 1) / slots;
        if (per_slot < waves_per_wg) waves_per_wg = per_slot < 4 ? 4 : per_slot;
        uint32_t grid = slots;
        const uint32_t need = (work + waves_per_wg - 1) / waves_per_wg;
        if (grid > need) grid = need;
        if (grid == 0) grid = 1;
        EriAdam8Hyper hh = *h;
        const float *dev_scale = nullptr;
        if (clip) {
            dev_scale = t->norm_last + 1;
            if (!scaled) { // the scale path is needed; neutral host-side factors
                hh.flags |= ERI_ADAM8_FLAG_GRAD_SCALE;
                hh.grad_scale = 1.0f;
            }
        }
        rc = eri::launch_step(g.dev, g.n, g.total_blocks, g.dtype, hh, ctx->image, dev_scale, grid, waves_per_wg * eri::kWave, ctx->cus, stream);
        if (rc) return hip_fail((hipError_t)rc, "adam8 step launch");
        if ((hh.flags & ERI_ADAM8_FLAG_EMA) && !eri::step_fuses_ema(g.total_blocks, g.dtype, hh, ctx->cus)) {
            // not the kernel that carries the EMA: this group's shadows join the plain sweep that follows the step
            for (uint32_t j = 0; j < g.n; ++j) {
                const eri::DevTensor &d = g.pinned[j];
                if (!d.shadow) continue;
                EriEmaTensor e;
                e.shadow = d.shadow;
                e.p = d.p;
                e.numel = d.numel;
                e.dtype_tag = eri::layout_param_bf16(g.dtype) ? ERI_DTYPE_BF16 : ERI_DTYPE_F32;
                e.reserved = 0;
                ema_rest.push_back(e);
            }
        }
    }
    if (!ema_rest.empty()) { // one sweep for all groups that did not carry their EMA, right behind the step
        rc = eri_ema_update_multi(ema_rest.data(), (uint32_t)ema_rest.size(), h->ema_decay, stream);
        if (rc) return rc;
    }
    return 0;
}

/* The launches of the gradient-norm pass over one table, or over two as if they were one (`also` may be null):
 * a sum-of-squares launch per group of rows, then one launch that adds the per-wave partial sums of all of them.
 * `partial` holds room for `pairs` {sum, count} pairs. */
static int grad_norm_launch(EriAdam8Table *t, EriAdam8Table *also, DeviceCtx *ctx, float max_norm, float denom_eps,
                            double *partial, uint32_t pairs, float *result, void *stream) {
    const uint32_t wpw = (uint32_t)eri::kNormWaves;
    const uint32_t grid_cap = ctx->cus * eri::kNormWavesPerCu / wpw; // persistent
    EriAdam8Table *tables[2] = {t, also};
    uint32_t grids[2][eri::kLayouts] = {{0, 0, 0}, {0, 0, 0}}, need = 0;
    for (int ti = 0; ti < 2; ++ti) {
        if (!tables[ti]) continue;
        for (int gi = 0; gi < eri::kLayouts; ++gi) {
            const auto &g = tables[ti]->groups[gi];
            if (g.n == 0) continue;
            const uint32_t work = g.total_blocks > g.n ? g.total_blocks : g.n;
            uint32_t grid = (work + wpw - 1) / wpw;
            if (grid > grid_cap) grid = grid_cap;
            grids[ti][gi] = grid;
            need += grid * wpw;
        }
    }
    if (need > pairs) {
        char buf[160];
        std::snprintf(buf, sizeof buf, "the gradient-norm pass of this table needs %u per-wave partial sums, the scratch holds %u",
                      need, pairs);
        return fail(ERI_ERR_TOO_LARGE, buf);
    }
    uint32_t off = 0;
    for (int ti = 0; ti < 2; ++ti) {
        if (!tables[ti]) continue;
        int rc = order_after_upload(tables[ti], stream);
        if (rc) return rc;
        for (int gi = 0; gi < eri::kLayouts; ++gi) {
            auto &g = tables[ti]->groups[gi];
            if (g.n == 0) continue;
            rc = eri::launch_grad_sumsq(g.dev, g.n, g.total_blocks, eri::layout_grad_bf16(g.dtype), partial + 2 * off, grids[ti][gi], stream);
            if (rc) return hip_fail((hipError_t)rc, "gradient sum-of-squares launch");
            off += grids[ti][gi] * wpw;
        }
    }
    t->n_partial = off;
    int rc = eri::launch_grad_norm_finish(partial, off, max_norm, denom_eps, result, stream);
    if (rc) return hip_fail((hipError_t)rc, "gradient norm launch");
    t->norm_last = result;
    if (also) also->norm_last = result;
    return 0;
}

static int grad_norm(EriAdam8Table *t, EriAdam8Table *also, float max_norm, float denom_eps, void *stream) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    if (also && also->device != t->device) return fail(ERI_ERR_ARG, "the two tables belong to different devices");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx_on(t->device, &ctx);
    if (rc) return rc;
    // per table one group per layout at most, and per wave a sum of squares and a count; room for two tables
    const uint32_t pairs = 2 * eri::kLayouts * ctx->cus * eri::kNormWavesPerCu;
    if (!t->partial) ERI_HIP(hipMalloc((void **)&t->partial, sizeof(double) * 2 * pairs));
    if (!t->norm_out) ERI_HIP(hipMalloc((void **)&t->norm_out, sizeof(float) * 4)); // norm, scale, 64-bit count
    return grad_norm_launch(t, also, ctx, max_norm, denom_eps, t->partial, pairs, t->norm_out, stream);
}

int eri_adam8_grad_norm(EriAdam8Table *t, float max_norm, float denom_eps, void *stream) {
    return grad_norm(t, nullptr, max_norm, denom_eps, stream);
}

int eri_adam8_grad_norm_joint(EriAdam8Table *t, EriAdam8Table *also, float max_norm, float denom_eps, void *stream) {
    if (!also) return fail(ERI_ERR_NULL, "the second table is NULL");
    if (also == t) return fail(ERI_ERR_ARG, "the two tables are the same");
    return grad_norm(t, also, max_norm, denom_eps, stream);
}

int eri_adam8_grad_norm_scale_ptr(const EriAdam8Table *t, const float **dev_scale) {
    if (!t || !dev_scale) return fail(ERI_ERR_NULL, "table or dev_scale is NULL");
    if (!t->norm_last) return fail(ERI_ERR_ARG, "no gradient norm has been computed for this table");
    *dev_scale = t->norm_last + 1;
    return 0;
}

int eri_adam8_grad_norm_static(EriAdam8Table *t, float max_norm, float denom_eps, void *result, void *stream) {
    if (!t || !result) return fail(ERI_ERR_NULL, "table or result is NULL");
    if ((uintptr_t)result & 7u) return fail(ERI_ERR_ALIGN, "result must be 8-byte aligned");
    int dev = -1;
    ERI_HIP(hipGetDevice(&dev));
    if (dev != t->device) return fail(ERI_ERR_ARG, "the table belongs to another device than the current one");
    // the device's context was made ready, scratch address included, when the table was created; it is read under
    // the lock that guards its creation, and nothing is created here
    DeviceCtx *ctx = &g_ctx[dev];
    {
        std::lock_guard<std::mutex> lk(g_ctx_mu);
        if (!ctx->ready || !ctx->scratch_ptr) return fail(ERI_ERR_INTERNAL, "the library was not initialised on this device");
    }
    return grad_norm_launch(t, nullptr, ctx, max_norm, denom_eps, ctx->scratch_ptr, kNormScratchPairs, static_cast<float *>(result), stream);
}

int eri_adam8_grad_norm_read(EriAdam8Table *t, float *norm, float *scale, void *stream) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    if (!t->norm_last) return fail(ERI_ERR_ARG, "no gradient norm has been computed for this table");
    float host[2] = {0.0f, 1.0f};
    ERI_HIP(hipMemcpyAsync(host, t->norm_last, sizeof host, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    ERI_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    if (norm) *norm = host[0];
    if (scale) *scale = host[1];
    return 0;
}

int eri_adam8_grad_nonfinite_read(EriAdam8Table *t, uint64_t *count, void *stream) {
    if (!t || !count) return fail(ERI_ERR_NULL, "table or count is NULL");
    if (!t->norm_last) return fail(ERI_ERR_ARG, "no gradient norm has been computed for this table");
    unsigned long long host = 0;
    ERI_HIP(hipMemcpyAsync(&host, t->norm_last + 2, sizeof host, hipMemcpyDeviceToHost, static_cast<hipStream_t>(stream)));
    ERI_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    *count = host;
    return 0;
}

int eri_adam8_traffic_probe(EriAdam8Table *t, void *stream) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    if (t->grads_only) return fail(ERI_ERR_ARG, "a gradient-only table serves eri_adam8_grad_norm only");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx_on(t->device, &ctx);
    if (rc) return rc;
    const auto &g = t->groups[eri::kLayoutBF16];
    if (g.n == 0 || g.total_blocks == 0) return fail(ERI_ERR_ARG, "the traffic probe needs full blocks of BF16 rows with BF16 gradients");
    rc = order_after_upload(t, stream);
    if (rc) return rc;
    rc = eri::launch_traffic_probe(g.dev, g.n, g.total_blocks, ctx->cus * ctx->wg_per_cu, stream);
    if (rc) return hip_fail((hipError_t)rc, "traffic probe launch");
    return 0;
}

int eri_adam8_quant_error(EriAdam8Table *t, const EriAdam8Hyper *h, void *stream) {
    if (!t || !h) return fail(ERI_ERR_NULL, "table or hyper is NULL");
    if (t->grads_only) return fail(ERI_ERR_ARG, "a gradient-only table serves eri_adam8_grad_norm only");
    if (h->mode != ERI_ADAM8_MODE_ERI && h->mode != ERI_ADAM8_MODE_L2)
        return fail(ERI_ERR_ARG, "the quantisation error pass knows the modes ERI and L2");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx_on(t->device, &ctx);
    if (rc) return rc;
    if (!t->qerr) ERI_HIP(hipMalloc((void **)&t->qerr, sizeof(double) * 2 * t->n));
    rc = order_after_upload(t, stream);
    if (rc) return rc;
    uint32_t off = 0;
    for (auto &g : t->groups) {
        if (g.n == 0) continue;
        EriAdam8Hyper hh = *h;
        const float *dev_scale = nullptr;
        if (hh.flags & ERI_ADAM8_FLAG_CLIP_FROM_TABLE) {
            if (!t->norm_last) return fail(ERI_ERR_ARG, "ERI_ADAM8_FLAG_CLIP_FROM_TABLE without a prior eri_adam8_grad_norm");
            dev_scale = t->norm_last + 1;
            if (!(hh.flags & ERI_ADAM8_FLAG_GRAD_SCALE)) {
                hh.flags |= ERI_ADAM8_FLAG_GRAD_SCALE;
                hh.grad_scale = 1.0f;
            }
        }
        uint32_t grid = (g.total_blocks + g.n + 3) / 4;
        if (grid > ctx->cus * 8) grid = ctx->cus * 8;
        rc = eri::launch_quant_error(g.dev, g.n, g.total_blocks, g.dtype, hh, ctx->image, dev_scale, t->qerr + 2 * off,
                                     grid, stream);
        if (rc) return hip_fail((hipError_t)rc, "quantisation error launch");
        off += g.n;
    }
    t->qerr_valid = true;
    return 0;
}

int eri_adam8_quant_error_read(EriAdam8Table *t, float *m_error, float *v_error, void *stream) {
    if (!t) return fail(ERI_ERR_NULL, "table is NULL");
    if (!t->qerr_valid) return fail(ERI_ERR_ARG, "no quantisation error has been computed for this table");
    std::vector<double> host(2 * (size_t)t->n);
    ERI_HIP(hipMemcpyAsync(host.data(), t->qerr, host.size() * sizeof(double), hipMemcpyDeviceToHost,
                           static_cast<hipStream_t>(stream)));
    ERI_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    double sm = 0.0, sv = 0.0;
    uint32_t off = 0;
    for (auto &g : t->groups)
        for (uint32_t j = 0; j < g.n; ++j, ++off) {
            const double n = (double)t->numel[g.src[j]];
            sm += host[2 * off] / n;     // per-tensor mean, adam8bit_enhanced.rs:100
            sv += host[2 * off + 1] / n;
        }
    if (m_error) *m_error = (float)(sm / (double)t->n); // mean over tensors, :319-324
    if (v_error) *v_error = (float)(sv / (double)t->n);
    return 0;
}

int eri_adam8_step_multi(const EriAdam8Tensor *rows, uint32_t n, const EriAdam8Hyper *h, void *stream) {
    struct Cache {
        EriAdam8Table *table = nullptr;
        std::vector<EriAdam8Tensor> last;
        ~Cache() { destroy_table(table); }
    };
    thread_local Cache cache;
    if (!rows || !h) return fail(ERI_ERR_NULL, "rows or hyper is NULL");
    int dev = 0;
    ERI_HIP(hipGetDevice(&dev));
    bool same_shape = cache.table && cache.table->n == n && cache.table->device == dev;
    if (same_shape)
        for (uint32_t i = 0; i < n && same_shape; ++i)
            same_shape = rows[i].numel == cache.table->numel[i] && layout_of(rows[i]) == cache.table->dtype[i];
    int rc = 0;
    if (!same_shape) {
        destroy_table(cache.table);
        cache.table = nullptr;
        cache.last.clear();
        rc = eri_adam8_table_create(rows, n, stream, &cache.table);
        if (rc) return rc;
        cache.last.assign(rows, rows + n);
    } else if (std::memcmp(cache.last.data(), rows, sizeof(EriAdam8Tensor) * n) != 0) {
        rc = eri_adam8_table_update(cache.table, rows, n, stream);
        if (rc) return rc;
        cache.last.assign(rows, rows + n);
    }
    return eri_adam8_step_table(cache.table, h, stream);
}

int eri_adam8_dequantize(const uint8_t *codes, const float *absmax, int signed_map, uint64_t numel, float *out,
                         void *stream) {
    if (!codes || !absmax || !out) return fail(ERI_ERR_NULL, "dequantize with NULL pointer");
    if (numel == 0) return fail(ERI_ERR_EMPTY, "Empty quantized data");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx(&ctx);
    if (rc) return rc;
    if ((rc = require_kernel_visible(codes, "dequantize: codes")) != 0) return rc;
    if ((rc = require_kernel_visible(absmax, "dequantize: absmax")) != 0) return rc;
    if ((rc = require_kernel_visible(out, "dequantize: out")) != 0) return rc;
    rc = eri::launch_dequantize(codes, absmax, signed_map, numel, out, ctx->image, stream);
    if (rc) return hip_fail((hipError_t)rc, "dequantize launch");
    return 0;
}

int eri_adam8_quantize(const float *x, int signed_map, uint64_t numel, uint8_t *codes, float *absmax, void *stream) {
    if (!x || !codes || !absmax) return fail(ERI_ERR_NULL, "quantize with NULL pointer");
    if (numel == 0) return fail(ERI_ERR_EMPTY, "Empty tensor for quantization");
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx(&ctx);
    if (rc) return rc;
    if ((rc = require_kernel_visible(x, "quantize: x")) != 0) return rc;
    if ((rc = require_kernel_visible(codes, "quantize: codes")) != 0) return rc;
    if ((rc = require_kernel_visible(absmax, "quantize: absmax")) != 0) return rc;
    rc = eri::launch_quantize(x, signed_map, numel, codes, absmax, ctx->image, stream);
    if (rc) return hip_fail((hipError_t)rc, "quantize launch");
    return 0;
}

} // extern "C"

// ---- plain sweeps: 32-bit AdamW, EMA ---------------------------------------------------------

namespace {

/* Device copies of the row tables of the plain sweeps, kept per calling thread.  An optimizer step can sweep
 * several row sets in turn (the shadows of the groups that do not carry the EMA inside the step kernel, then the
 * parameters outside the 8-bit table), the same sets step after step, so the last four distinct sets are kept:
 * rows found in one of them are not uploaded again.  A set is uploaded through its own pinned mirror, whose
 * previous copy is waited for before it is overwritten; a set that is used on another stream than the one it
 * was uploaded on is ordered after the upload by an event wait on that stream. */
struct ElemCache {
    struct Group {
        eri::ElemRow *dev = nullptr, *pinned = nullptr;
        uint32_t cap = 0, n = 0;
    };
    struct Slot {
        Group groups[2]; // F32, BF16
        hipEvent_t ev = nullptr;
        bool pending = false;
        void *stream = nullptr; // of the last upload
        uint64_t used = 0;
        void drop() {
            if (pending && ev) (void)hipEventSynchronize(ev);
            pending = false;
            for (auto &g : groups) {
                if (g.dev) (void)hipFree(g.dev);
                if (g.pinned) (void)hipHostFree(g.pinned);
                g.dev = g.pinned = nullptr;
                g.cap = g.n = 0;
            }
            if (ev) (void)hipEventDestroy(ev);
            ev = nullptr;
            used = 0;
        }
    };
    static constexpr int kSlots = 4;
    Slot slots[kSlots];
    std::vector<eri::ElemRow> rows[2]; // the rows of the call at hand: F32, BF16
    uint64_t tick = 0;
    int device = -1;
    ~ElemCache() {
        for (auto &sl : slots) sl.drop();
    }
    bool holds(const Slot &sl) const {
        for (int gi = 0; gi < 2; ++gi) {
            const uint32_t n = (uint32_t)rows[gi].size();
            if (sl.groups[gi].n != n) return false;
            if (n && std::memcmp(sl.groups[gi].pinned, rows[gi].data(), n * sizeof(eri::ElemRow)) != 0) return false;
        }
        return sl.used != 0;
    }
    int sync(void *stream, uint32_t cus, int (*launch)(const eri::ElemRow *, uint32_t, uint32_t, int, uint32_t, void *, const void *),
             const void *extra) {
        int dev = 0;
        ERI_HIP(hipGetDevice(&dev));
        if (dev != device) { // the thread moved to another device: nothing cached is an address there
            for (auto &sl : slots) sl.drop();
            device = dev;
        }
        Slot *sl = nullptr;
        for (auto &c : slots)
            if (holds(c)) sl = &c;
        if (sl) {
            if (sl->pending && hipEventQuery(sl->ev) == hipSuccess) sl->pending = false;
            (void)hipGetLastError(); // hipErrorNotReady of the query is not an error
            if (sl->pending && stream != sl->stream) { // uploaded on another stream and perhaps still on its way
                hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
                if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &cs) != hipSuccess) {
                    (void)hipGetLastError();
                    cs = hipStreamCaptureStatusNone;
                }
                if (cs == hipStreamCaptureStatusActive) { // a capture cannot wait for an event from outside it
                    ERI_HIP(hipEventSynchronize(sl->ev));
                    sl->pending = false;
                } else {
                    ERI_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), sl->ev, 0));
                }
            }
        } else {
            sl = &slots[0];
            for (auto &c : slots)
                if (c.used < sl->used) sl = &c;
            if (!sl->ev) ERI_HIP(hipEventCreateWithFlags(&sl->ev, hipEventDisableTiming));
            if (sl->pending) { // the mirror may still be the source of the slot's last copy
                ERI_HIP(hipEventSynchronize(sl->ev));
                sl->pending = false;
            }
            sl->used = 0; // not a set to come back to until the upload below is complete
            for (int gi = 0; gi < 2; ++gi) {
                Group &g = sl->groups[gi];
                const uint32_t n = (uint32_t)rows[gi].size();
                g.n = 0;
                if (n == 0) continue;
                if (g.cap < n) {
                    if (g.dev) (void)hipFree(g.dev);
                    if (g.pinned) (void)hipHostFree(g.pinned);
                    g.dev = g.pinned = nullptr;
                    g.cap = 0; // stays 0 if an allocation below fails: the next call starts over
                    const uint32_t cap = n + n / 2 + 16;
                    ERI_HIP(hipMalloc((void **)&g.dev, sizeof(eri::ElemRow) * cap));
                    ERI_HIP(hipHostMalloc((void **)&g.pinned, sizeof(eri::ElemRow) * cap, hipHostMallocDefault));
                    g.cap = cap;
                }
                std::memcpy(g.pinned, rows[gi].data(), n * sizeof(eri::ElemRow));
                ERI_HIP(hipMemcpyAsync(g.dev, g.pinned, n * sizeof(eri::ElemRow), hipMemcpyHostToDevice,
                                       static_cast<hipStream_t>(stream)));
                g.n = n;
            }
            ERI_HIP(hipEventRecord(sl->ev, static_cast<hipStream_t>(stream)));
            sl->pending = true;
            sl->stream = stream;
        }
        sl->used = ++tick;
        for (int gi = 0; gi < 2; ++gi) {
            const Group &g = sl->groups[gi];
            const uint32_t n = g.n;
            if (n == 0) continue;
            const eri::ElemRow &last = rows[gi].back();
            const uint32_t total = last.full_start + (uint32_t)(last.numel / eri::kBlock);
            const uint32_t work = total > n ? total : n;
            uint32_t grid = (work + 3) / 4;
            if (grid > cus * 16) grid = cus * 16;
            int rc = launch(g.dev, n, total, gi == 0 ? ERI_DTYPE_F32 : ERI_DTYPE_BF16, grid, stream, extra);
            if (rc) return hip_fail((hipError_t)rc, "element-wise sweep launch");
        }
        return 0;
    }
};

int check_elem(const void *a, const void *b, uint64_t numel, int dtype, uint32_t i, uint64_t &blocks) {
    char buf[128];
    if (!a || !b) { std::snprintf(buf, sizeof buf, "row %u: NULL pointer", i); return fail(ERI_ERR_NULL, buf); }
    if (numel == 0) { std::snprintf(buf, sizeof buf, "row %u: empty tensor", i); return fail(ERI_ERR_EMPTY, buf); }
    if (dtype != ERI_DTYPE_F32 && dtype != ERI_DTYPE_BF16) { std::snprintf(buf, sizeof buf, "row %u: unsupported dtype tag %d", i, dtype); return fail(ERI_ERR_DTYPE, buf); }
    if (((uintptr_t)a | (uintptr_t)b) & 15u) { std::snprintf(buf, sizeof buf, "row %u: pointers must be 16-byte aligned", i); return fail(ERI_ERR_ALIGN, buf); }
    blocks += numel / eri::kBlock;
    if (blocks > 0x7fffffffull) return fail(ERI_ERR_TOO_LARGE, "more than 2^31 - 1 blocks in one call");
    return 0;
}

struct AdamW32Extra {
    EriAdamW32Hyper h;
    bool scaled;            // gradients are multiplied by (grad_scale * row scale) * (*dev_scale)
    float grad_scale;
    const float *dev_scale; // device, or null for 1
};
int adamw32_launch(const eri::ElemRow *rows, uint32_t n, uint32_t total, int dtype, uint32_t grid, void *stream, const void *extra) {
    const AdamW32Extra &x = *static_cast<const AdamW32Extra *>(extra);
    return eri::launch_adamw32(rows, n, total, dtype, x.h, x.scaled, x.grad_scale, x.dev_scale, grid, stream);
}
int ema_launch(const eri::ElemRow *rows, uint32_t n, uint32_t total, int dtype, uint32_t grid, void *stream, const void *extra) {
    return eri::launch_ema(rows, n, total, dtype, *static_cast<const float *>(extra), grid, stream);
}

} // namespace

extern "C" {

static int adamw32_step(const EriAdamW32Tensor *rows, uint32_t n, const EriAdamW32Hyper *hyper, bool scaled, float grad_scale,
                        const float *dev_scale, void *stream) {
    if (!rows || !hyper) return fail(ERI_ERR_NULL, "rows or hyper is NULL");
    if (n == 0) return fail(ERI_ERR_ARG, "no rows");
    thread_local ElemCache cache;
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx(&ctx);
    for (auto &g : cache.rows) g.clear();
    uint64_t blocks = 0;
    uint32_t starts[2] = {0, 0};
    for (uint32_t i = 0; i < n; ++i) {
        const EriAdamW32Tensor &r = rows[i];
        int e = check_elem(r.p, r.g, r.numel, r.dtype_tag, i, blocks);
        if (e) return e;
        if (!r.m || !r.v) return fail(ERI_ERR_NULL, "moment pointer is NULL");
        if (((uintptr_t)r.m | (uintptr_t)r.v) & 15u) return fail(ERI_ERR_ALIGN, "moment pointers must be 16-byte aligned");
        const int gi = r.dtype_tag == ERI_DTYPE_F32 ? 0 : 1;
        eri::ElemRow d;
        if ((uintptr_t)r.master & 15u) return fail(ERI_ERR_ALIGN, "master pointer must be 16-byte aligned");
        d.a = r.p; d.b = r.g; d.c = r.m; d.d = r.v; d.e = r.master; d.numel = r.numel; d.full_start = starts[gi];
        d.scale = r.grad_scale == 0.0f ? 1.0f : r.grad_scale; // a zeroed row: no multiplier
        starts[gi] += (uint32_t)(r.numel / eri::kBlock);
        cache.rows[gi].push_back(d);
    }
    if (rc) return rc;
    AdamW32Extra x;
    x.h = *hyper;
    x.scaled = scaled;
    x.grad_scale = grad_scale;
    x.dev_scale = dev_scale;
    return cache.sync(stream, ctx->cus, adamw32_launch, &x);
}

int eri_adamw32_step_multi(const EriAdamW32Tensor *rows, uint32_t n, const EriAdamW32Hyper *hyper, void *stream) {
    return adamw32_step(rows, n, hyper, false, 1.0f, nullptr, stream);
}

int eri_adamw32_step_multi_scaled(const EriAdamW32Tensor *rows, uint32_t n, const EriAdamW32Hyper *hyper, float grad_scale,
                                  const float *dev_scale, void *stream) {
    return adamw32_step(rows, n, hyper, true, grad_scale, dev_scale, stream);
}

int eri_ema_update_multi(const EriEmaTensor *rows, uint32_t n, float decay, void *stream) {
    if (!rows) return fail(ERI_ERR_NULL, "rows is NULL");
    if (n == 0) return fail(ERI_ERR_ARG, "no rows");
    thread_local ElemCache cache;
    DeviceCtx *ctx = nullptr;
    int rc = get_ctx(&ctx);
    for (auto &g : cache.rows) g.clear();
    uint64_t blocks = 0;
    uint32_t starts[2] = {0, 0};
    for (uint32_t i = 0; i < n; ++i) {
        const EriEmaTensor &r = rows[i];
        int e = check_elem(r.shadow, r.p, r.numel, r.dtype_tag, i, blocks);
        if (e) return e;
        const int gi = r.dtype_tag == ERI_DTYPE_F32 ? 0 : 1;
        eri::ElemRow d;
        d.a = r.shadow; d.b = r.p; d.c = nullptr; d.d = nullptr; d.e = nullptr; d.numel = r.numel; d.full_start = starts[gi]; d.scale = 0.0f;
        starts[gi] += (uint32_t)(r.numel / eri::kBlock);
        cache.rows[gi].push_back(d);
    }
    if (rc) return rc;
    return cache.sync(stream, ctx->cus, ema_launch, &decay);
}

} // extern "C"
