/*
 * Host layer of the 8-bit Adam objects (include/eri_adam8bit.h), written against the C ABI of
 * include/eri_optim8.h only: no HIP headers, no torch.  It holds what the reference's Rust structs
 * hold -- the parameter handles, hyper-parameters, step counter and per-parameter 8-bit state --
 * plus the cached device launch table, and turns every step() into one eri_adam8_step_table call.
 *
 * Reference structures mirrored here:
 *   Adam8bit / Adam8bitConfig / OptimizerState   src/trainers/adam8bit_enhanced.rs:10-27,372-404
 *   Adam8bit (functional) / Adam8bitState        src/trainers/adam8bit.rs:15-47
 */
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <string_view>
#include <vector>

#include "../../include/eri_adam8bit.h"

namespace {

constexpr uint64_t kBlock = ERI_ADAM8_BLOCK;

uint64_t blocks_of(uint64_t numel) { return (numel + kBlock - 1) / kBlock; }
uint64_t align256(uint64_t n) { return (n + 255) & ~(uint64_t)255; }

int fail(int code, const std::string &msg) {
    eri_set_last_error(msg.c_str());
    return code;
}

/* uint8 codes and per-block absmax of both moments, in one device allocation or one piece of a memory pool. */
struct State8 {
    void *base = nullptr;
    EriHipPool *pool = nullptr; // the pool the piece came from and goes back to (not owned), or null
    uint64_t total = 0;         // bytes of the piece
    uint8_t *m = nullptr, *v = nullptr;
    float *absmax_m = nullptr, *absmax_v = nullptr;
    uint64_t numel = 0;

    int allocate(uint64_t n, void *stream, EriHipPool *from = nullptr, uint32_t lane = 0) {
        release();
        const uint64_t nb = blocks_of(n);
        const uint64_t o_v = align256(n), o_am = o_v + align256(n), o_av = o_am + align256(nb * 4);
        const uint64_t bytes = o_av + align256(nb * 4);
        int dev = 0;
        int rc = eri_hip_get_device(&dev);
        if (rc) return rc;
        // out of a pool the piece is cleared on the optimizer's stream (state_init below overwrites it anyway)
        rc = from ? eri_hip_pool_alloc_zeroed_async(from, lane, bytes, stream, &base) : eri_hip_malloc_zeroed(dev, bytes, &base);
        if (rc) return rc;
        if (from) eri_hip_pool_retain(from); // the piece goes back to it, also if the caller destroys the pool first
        pool = from;
        total = bytes;
        char *b = static_cast<char *>(base);
        m = reinterpret_cast<uint8_t *>(b);
        v = reinterpret_cast<uint8_t *>(b + o_v);
        absmax_m = reinterpret_cast<float *>(b + o_am);
        absmax_v = reinterpret_cast<float *>(b + o_av);
        numel = n;
        // the state of a zeros tensor (adam8bit_enhanced.rs:179-197)
        return eri_adam8_state_init(m, v, absmax_m, absmax_v, n, stream);
    }
    /* A pooled piece goes back to its pool, where the next state of the same size takes it (loading a checkpoint
     * replaces every state by one of its size).  The state holds the pool (eri_hip_pool_retain) until then. */
    void release() {
        if (base && pool) {
            eri_hip_pool_release(pool, base, total);
            eri_hip_pool_unretain(pool);
        } else if (base) {
            eri_hip_free(base);
        }
        base = nullptr;
        pool = nullptr;
        total = 0;
        m = v = nullptr;
        absmax_m = absmax_v = nullptr;
        numel = 0;
    }
    uint64_t nbytes() const { return numel ? 2 * numel + 8 * blocks_of(numel) : 0; }
    ~State8() { release(); }
    State8() = default;
    State8(const State8 &) = delete;
    State8 &operator=(const State8 &) = delete;
};

/* fp32 moments of a parameter that is kept out of the 8-bit format (min_8bit_size), in one device
 * allocation; zero-filled = the state of a zeros tensor. */
struct State32 {
    void *base = nullptr;
    float *m = nullptr, *v = nullptr;
    uint64_t numel = 0;
    int allocate(uint64_t n) {
        release();
        int dev = 0;
        int rc = eri_hip_get_device(&dev);
        if (rc) return rc;
        const uint64_t half = align256(n * 4);
        rc = eri_hip_malloc_zeroed(dev, 2 * half, &base);
        if (rc) return rc;
        m = static_cast<float *>(base);
        v = reinterpret_cast<float *>(static_cast<char *>(base) + half);
        numel = n;
        return 0;
    }
    void release() {
        if (base) eri_hip_free(base);
        base = nullptr;
        m = v = nullptr;
        numel = 0;
    }
    uint64_t nbytes() const { return 8 * numel; }
    ~State32() { release(); }
    State32() = default;
    State32(const State32 &) = delete;
    State32 &operator=(const State32 &) = delete;
};

// ---- a very small safetensors reader / writer ------------------------------------------------

struct StEntry {
    std::string dtype;
    std::vector<uint64_t> shape;
    uint64_t begin = 0, end = 0;
};

struct StFile {
    std::map<std::string, std::string> metadata;
    std::map<std::string, StEntry> tensors;
    uint64_t data_start = 0; // file offset of the byte that data_offsets count from
};

struct JsonCursor {
    const char *p, *e;
    bool ok = true;
    void ws() { while (p < e && (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r')) ++p; }
    bool eat(char c) {
        ws();
        if (p < e && *p == c) { ++p; return true; }
        ok = false;
        return false;
    }
    bool peek(char c) { ws(); return p < e && *p == c; }
    std::string str() {
        std::string out;
        if (!eat('"')) return out;
        while (p < e && *p != '"') {
            if (*p == '\\' && p + 1 < e) { ++p; }
            out.push_back(*p++);
        }
        if (p >= e) { ok = false; return out; }
        ++p;
        return out;
    }
    uint64_t num() {
        ws();
        uint64_t v = 0;
        bool any = false;
        while (p < e && *p >= '0' && *p <= '9') { v = v * 10 + (uint64_t)(*p++ - '0'); any = true; }
        if (!any) ok = false;
        return v;
    }
};

/* Reads and checks the header of an open safetensors file; tensor bytes stay in the file. */
bool parse_safetensors(std::ifstream &f, StFile &out, std::string &why) {
    f.seekg(0, std::ios::end);
    const std::streamoff end_pos = f.tellg();
    f.seekg(0, std::ios::beg);
    if (!f || end_pos < 8) { why = "file shorter than its header length"; return false; }
    const uint64_t size = (uint64_t)end_pos;
    uint64_t hlen = 0;
    f.read(reinterpret_cast<char *>(&hlen), 8);
    if (!f || hlen > size - 8) { why = "header length exceeds the file"; return false; }
    std::vector<char> raw((size_t)hlen);
    f.read(raw.data(), (std::streamsize)hlen);
    if (!f) { why = "header cannot be read"; return false; }
    JsonCursor c{raw.data(), raw.data() + hlen};
    if (!c.eat('{')) { why = "header is not a JSON object"; return false; }
    bool first = true;
    while (c.ok && !c.peek('}')) {
        if (!first && !c.eat(',')) break;
        first = false;
        const std::string key = c.str();
        if (!c.eat(':') || !c.eat('{')) break;
        bool f2 = true;
        StEntry ent;
        while (c.ok && !c.peek('}')) {
            if (!f2 && !c.eat(',')) break;
            f2 = false;
            const std::string k2 = c.str();
            if (!c.eat(':')) break;
            if (key == "__metadata__") {
                out.metadata[k2] = c.str();
            } else if (k2 == "dtype") {
                ent.dtype = c.str();
            } else if (k2 == "shape" || k2 == "data_offsets") {
                std::vector<uint64_t> vals;
                if (!c.eat('[')) break;
                while (c.ok && !c.peek(']')) {
                    if (!vals.empty() && !c.eat(',')) break;
                    vals.push_back(c.num());
                }
                c.eat(']');
                if (k2 == "shape") ent.shape = vals;
                else if (vals.size() == 2) { ent.begin = vals[0]; ent.end = vals[1]; }
                else c.ok = false;
            } else {
                c.ok = false;
            }
        }
        c.eat('}');
        if (key != "__metadata__") out.tensors[key] = ent;
    }
    if (!c.ok || !c.eat('}')) { why = "malformed header"; return false; }
    out.data_start = 8 + hlen;
    for (auto &kv : out.tensors)
        if (kv.second.end < kv.second.begin || kv.second.end > size - out.data_start) {
            why = "tensor '" + kv.first + "' points outside the file";
            return false;
        }
    return true;
}

/* The header is complete before any tensor byte exists: sizes alone fix the offsets, so the caller
 * can stream the tensors behind it in the order it added them. */
struct StWriter {
    std::ostringstream header;
    uint64_t offset = 0;
    void begin(const std::map<std::string, std::string> &meta) {
        header << "{\"__metadata__\":{";
        bool f = true;
        for (auto &kv : meta) {
            header << (f ? "" : ",") << "\"" << kv.first << "\":\"" << kv.second << "\"";
            f = false;
        }
        header << "}";
    }
    void add(const std::string &name, const char *dtype, uint64_t count, uint64_t bytes) {
        header << ",\"" << name << "\":{\"dtype\":\"" << dtype << "\",\"shape\":[" << count << "],\"data_offsets\":["
               << offset << "," << offset + bytes << "]}";
        offset += bytes;
    }
    bool write_header(std::ofstream &f) {
        header << "}";
        std::string h = header.str();
        while (h.size() % 8) h.push_back(' ');
        const uint64_t hl = h.size();
        f.write(reinterpret_cast<const char *>(&hl), 8);
        f.write(h.data(), (std::streamsize)h.size());
        return (bool)f;
    }
};

/* Pinned host memory in two halves, through which state moves between the device and a file in
 * bounded pieces: one half is in a device copy while the other is read or written. */
struct Bounce {
    static constexpr uint64_t kHalf = (uint64_t)32 << 20;
    char *host = nullptr;
    int which = 0;
    int ensure() {
        if (host) return 0;
        host = static_cast<char *>(eri_hip_host_alloc(2 * kHalf));
        return host ? 0 : ERI_ERR_INTERNAL; // the allocator has set the message
    }
    char *next() { which ^= 1; return host + which * kHalf; }
    ~Bounce() { if (host) eri_hip_host_free(host); }
};

/* device -> file.  The copy of piece i+1 is queued before piece i is written. */
int stream_out(std::ofstream &f, const void *dev, uint64_t bytes, Bounce &b, void *stream) {
    const char *src = static_cast<const char *>(dev);
    char *cur = nullptr;
    uint64_t cur_n = 0;
    for (uint64_t done = 0; done < bytes || cur;) {
        char *nxt = nullptr;
        uint64_t nxt_n = 0;
        if (done < bytes) {
            nxt = b.next();
            nxt_n = bytes - done < Bounce::kHalf ? bytes - done : Bounce::kHalf;
            int rc = eri_hip_memcpy_async(nxt, src + done, nxt_n, 2, stream);
            if (rc) return rc;
            done += nxt_n;
        }
        if (cur) {
            f.write(cur, (std::streamsize)cur_n);
            if (!f) return fail(ERI_ERR_ARG, "InvalidOperation: Failed to save optimizer: write failed");
        }
        if (nxt) {
            int rc = eri_hip_stream_sync(stream);
            if (rc) return rc;
        }
        cur = nxt;
        cur_n = nxt_n;
    }
    return 0;
}

/* file -> device.  Piece i+1 is read from the file while piece i is in its copy. */
int stream_in(std::ifstream &f, uint64_t file_offset, void *dev, uint64_t bytes, Bounce &b, void *stream) {
    f.seekg((std::streamoff)file_offset, std::ios::beg);
    char *dst = static_cast<char *>(dev);
    for (uint64_t done = 0; done < bytes;) {
        char *buf = b.next();
        const uint64_t n = bytes - done < Bounce::kHalf ? bytes - done : Bounce::kHalf;
        f.read(buf, (std::streamsize)n);
        if (!f) return fail(ERI_ERR_ARG, "InvalidOperation: Failed to read optimizer: file ends inside a tensor");
        int rc = eri_hip_stream_sync(stream); // the other half's copy; this half's was waited for a round ago
        if (rc) return rc;
        rc = eri_hip_memcpy_async(dst + done, buf, n, 1, stream);
        if (rc) return rc;
        done += n;
    }
    return eri_hip_stream_sync(stream);
}

} // namespace

// ---------------------------------------------------------------------------------------------
// Parameter
// ---------------------------------------------------------------------------------------------

struct EriParameter {
    void *data = nullptr;
    const void *grad = nullptr;
    uint64_t numel = 0;
    int32_t dtype = 0;
    int32_t grad_dtype = 0; // dtype of *grad: the parameter's, or F32 for a BF16 parameter
    int refs = 1;
};

// ---------------------------------------------------------------------------------------------
// EMAModel: named shadows (defined here because the optimizer below can carry one in its step)
// ---------------------------------------------------------------------------------------------

struct EriEmaModel {
    struct Shadow {
        void *data = nullptr;
        uint64_t numel = 0;
        int32_t dtype = 0;
    };
    float decay = 0.999f, power = 1.0f;
    bool bias_correction = true;
    uint64_t step = 0;
    void *stream = nullptr;
    std::map<std::string, Shadow> shadows;
    std::vector<EriEmaTensor> rows; // reused between updates
    ~EriEmaModel() {
        for (auto &kv : shadows)
            if (kv.second.data) eri_hip_free(kv.second.data);
    }
};

namespace {

uint64_t elem_bytes(int32_t dtype) { return dtype == ERI_DTYPE_F32 ? 4 : 2; }

// a fresh shadow holding a copy of the parameter (ema_enhanced.rs:72-73,100-103)
int ema_adopt(EriEmaModel *e, const std::string &name, const EriParameter *p) {
    if (!p || !p->data) return fail(ERI_ERR_NULL, "parameter without data: " + name);
    if (p->numel == 0) return fail(ERI_ERR_EMPTY, "empty parameter: " + name);
    if (p->dtype != ERI_DTYPE_F32 && p->dtype != ERI_DTYPE_BF16) return fail(ERI_ERR_DTYPE, "Unsupported: EMA takes F32 or BF16 parameters");
    EriEmaModel::Shadow &s = e->shadows[name];
    const uint64_t bytes = p->numel * elem_bytes(p->dtype);
    if (!s.data || s.numel != p->numel || s.dtype != p->dtype) {
        if (s.data) eri_hip_free(s.data);
        s = EriEmaModel::Shadow();
        int dev = 0;
        int rc = eri_hip_get_device(&dev);
        if (!rc) rc = eri_hip_malloc_zeroed(dev, bytes, &s.data);
        if (rc) {
            e->shadows.erase(name);
            return rc;
        }
        s.numel = p->numel;
        s.dtype = p->dtype;
    }
    return eri_hip_memcpy_async(s.data, p->data, bytes, 3, e->stream);
}

} // namespace

// ---------------------------------------------------------------------------------------------
// Adam8bit over a parameter list
// ---------------------------------------------------------------------------------------------

struct EriAdam8bit {
    std::vector<EriParameter *> params;
    double lr = 1e-3, beta1 = 0.9, beta2 = 0.999, eps = 1e-8, wd = 0.01;
    uint64_t step = 0;
    // bf16 parameters come out with the reference's bits unless the caller trades that for the last 0.6-0.9 %
    uint32_t flags = ERI_ADAM8_FLAG_EXACT_PARAM;
    int mode = ERI_ADAM8_MODE_ERI;
    float grad_scale = 1.0f;
    float max_grad_norm = 0.0f, clip_denom_eps = 0.0f;
    bool track_qerr = false, have_qerr = false;
    std::vector<float> param_scale;
    std::vector<std::unique_ptr<State8>> states; // index = parameter index; null before the first step
    std::vector<std::unique_ptr<State32>> states32; // fp32 moments of the parameters below min_8bit_size
    uint64_t min_8bit_size = 0;                   // 0 = every parameter takes the 8-bit format
    EriEmaModel *ema = nullptr;                   // attached EMA model (not owned), updated inside step()
    std::vector<std::string> ema_names;           // its name for each parameter
    void *stream = nullptr;
    EriHipPool *state_pool = nullptr;        // where states not yet created will come from (not owned)
    uint32_t state_lane = 0;
    EriAdam8Table *table = nullptr;
    std::vector<uint32_t> table_ids;         // parameter indices the table was built for
    std::vector<EriAdam8Tensor> table_rows;  // rows as last uploaded
    EriAdam8Table *grad_table = nullptr;     // gradients of the tensors kept in 32-bit moments, for the global norm
    std::vector<EriAdam8Tensor> grad_rows;
    EriAdam8Table *norm_table = nullptr;     // the table that holds the last norm: table or grad_table (not owned twice)
};

/* One named state of the functional flavour with its own one-row launch table: updates of many
 * names in turn then cost a pointer comparison each, not a table rebuild. */
struct FnState : State8 {
    EriAdam8Table *table = nullptr;
    EriAdam8Tensor row;
    uint64_t queued_in = 0; // generation of the batch that holds a row of this state
    FnState() { std::memset(&row, 0, sizeof row); }
    ~FnState() {
        if (table) eri_adam8_table_destroy(table);
    }
};

struct EriAdam8bitFn {
    double lr = 1e-4, beta1 = 0.9, beta2 = 0.999, eps = 1e-8, wd = 0.01;
    uint64_t step = 0;
    void *stream = nullptr;
    EriHipPool *state_pool = nullptr; // where states not yet created will come from (not owned)
    uint32_t state_lane = 0;
    std::map<std::string, std::unique_ptr<FnState>, std::less<>> states;
    // Batching: update() calls queue rows, one launch over all of them runs at the next flush.
    bool batching = false;
    uint64_t generation = 1;                 // of the batch being collected
    std::vector<EriAdam8Tensor> pending;     // rows in call order
    std::vector<std::pair<const std::string *, FnState *>> pending_who;
    std::vector<std::pair<const std::string *, FnState *>> last_order; // names of the last flush, in order
    // Launch tables of the last two distinct sets of rows.  update() returns a new tensor per call
    // (adam8bit.rs:205-207), so the pointers of one flush differ from those of the flush before; a trainer
    // that drops the old tensor as it takes the new one gets the old addresses back from its allocator, and
    // the row sets alternate between two.  Two tables then serve every flush without an upload.
    struct TableSlot {
        EriAdam8Table *table = nullptr;
        std::vector<EriAdam8Tensor> rows; // as last uploaded
        uint64_t used = 0;                // flush counter of the last use
    } slots[2];
    uint64_t flushes = 0;
    uint64_t uploads = 0; // flushes that had to create or re-upload a table
    ~EriAdam8bitFn() {
        for (auto &sl : slots)
            if (sl.table) eri_adam8_table_destroy(sl.table);
    }
};

namespace {
int fn_flush(EriAdam8bitFn *o);
}

extern "C" {

int eri_param_create(void *data, uint64_t numel, int dtype_tag, EriParameter **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (!data) return fail(ERI_ERR_NULL, "parameter data is NULL");
    if (dtype_tag != ERI_DTYPE_F32 && dtype_tag != ERI_DTYPE_BF16)
        return fail(ERI_ERR_DTYPE, "Unsupported: 8-bit Adam takes F32 or BF16 parameters");
    EriParameter *p = new EriParameter();
    p->data = data;
    p->numel = numel;
    p->dtype = dtype_tag;
    p->grad_dtype = dtype_tag;
    *out = p;
    return 0;
}

int eri_param_set_grad(EriParameter *param, const void *grad) {
    if (!param) return fail(ERI_ERR_NULL, "param is NULL");
    param->grad = grad;
    param->grad_dtype = param->dtype;
    return 0;
}

int eri_param_set_grad_typed(EriParameter *param, const void *grad, int grad_dtype_tag) {
    if (!param) return fail(ERI_ERR_NULL, "param is NULL");
    if (grad_dtype_tag != param->dtype && !(param->dtype == ERI_DTYPE_BF16 && grad_dtype_tag == ERI_DTYPE_F32))
        return fail(ERI_ERR_DTYPE, "Unsupported: a gradient has the dtype of its parameter, or F32 for a BF16 parameter");
    param->grad = grad;
    param->grad_dtype = grad_dtype_tag;
    return 0;
}

int eri_param_set_data(EriParameter *param, void *data) {
    if (!param || !data) return fail(ERI_ERR_NULL, "param or data is NULL");
    param->data = data;
    return 0;
}

int eri_param_retain(EriParameter *param) {
    if (!param) return fail(ERI_ERR_NULL, "param is NULL");
    ++param->refs;
    return 0;
}

int eri_param_release(EriParameter *param) {
    if (!param) return 0;
    if (--param->refs == 0) delete param;
    return 0;
}

void eri_adam8bit_config_default(EriAdam8bitConfig *cfg) {
    if (!cfg) return;
    cfg->lr = 1e-3;
    cfg->beta1 = 0.9;
    cfg->beta2 = 0.999;
    cfg->eps = 1e-8;
    cfg->weight_decay = 0.01;
    cfg->amsgrad = 0;
    cfg->block_wise = 1;
    cfg->percentile_clipping = 99;
}

int eri_adam8bit_new(EriParameter *const *params, uint32_t n, const EriAdam8bitConfig *cfg, void *stream,
                     EriAdam8bit **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (n && !params) return fail(ERI_ERR_NULL, "params is NULL");
    EriAdam8bitConfig c;
    eri_adam8bit_config_default(&c);
    if (cfg) c = *cfg;
    for (uint32_t i = 0; i < n; ++i)
        if (!params[i]) return fail(ERI_ERR_NULL, "a parameter handle is NULL");
    EriAdam8bit *o = new EriAdam8bit();
    o->lr = c.lr;
    o->beta1 = c.beta1;
    o->beta2 = c.beta2;
    o->eps = c.eps;
    o->wd = c.weight_decay;
    o->stream = stream;
    o->params.assign(params, params + n);
    for (auto *p : o->params) ++p->refs; // the optimizer holds clones of the handles (:222-223)
    o->states.resize(n);
    o->states32.resize(n);
    o->param_scale.assign(n, 1.0f);
    *out = o;
    return 0;
}

int eri_adam8bit_destroy(EriAdam8bit *o) {
    if (!o) return 0;
    if (o->table) eri_adam8_table_destroy(o->table);
    if (o->grad_table) eri_adam8_table_destroy(o->grad_table);
    for (auto *p : o->params) eri_param_release(p);
    delete o;
    return 0;
}

static int adam8bit_step_impl(EriAdam8bit *o, uint32_t *skipped);

/* The part of an attached EMA model's update that the 8-bit step did not do itself. */
static int adam8bit_ema_rest(EriAdam8bit *o, const std::vector<EriEmaTensor> &others, const std::vector<uint32_t> &fresh,
                             float decay) {
    if (!o->ema) return 0;
    if (!others.empty()) {
        int rc = eri_ema_update_multi(others.data(), (uint32_t)others.size(), decay, o->stream);
        if (rc) return rc;
    }
    for (uint32_t i : fresh) {
        int rc = ema_adopt(o->ema, o->ema_names[i], o->params[i]);
        if (rc) return rc;
    }
    return 0;
}

int eri_adam8bit_step(EriAdam8bit *o, uint32_t *skipped) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    const uint64_t before = o->step, ema_before = o->ema ? o->ema->step : 0;
    const int rc = adam8bit_step_impl(o, skipped);
    if (rc) { // a refused step counts for nothing
        o->step = before;
        if (o->ema) o->ema->step = ema_before;
    }
    return rc;
}

static int adam8bit_step_impl(EriAdam8bit *o, uint32_t *skipped) {
    o->step += 1; // :203
    uint32_t skip = 0;
    std::vector<uint32_t> ids;
    std::vector<EriAdam8Tensor> rows;
    std::vector<EriAdamW32Tensor> rows32;
    uint64_t start = 0;
    bool scaled = o->grad_scale != 1.0f;
    for (uint32_t i = 0; i < o->params.size(); ++i) {
        EriParameter *p = o->params[i];
        if (!p->grad) { // :237-240
            std::fprintf(stderr, "Warning: No gradient for param_%u\n", i);
            ++skip;
            continue;
        }
        if (p->numel == 0) return fail(ERI_ERR_EMPTY, "InvalidOperation: Empty tensor for quantization");
        // min_8bit_size (pipeline_flux_lora_1024.rs:451): a short tensor keeps fp32 moments and takes the same
        // update without the quantiser, unless it already has an 8-bit state or its gradient is of another dtype
        const bool small = o->states32[i] || (o->min_8bit_size && p->numel < o->min_8bit_size && !o->states[i] &&
                                              p->grad_dtype == p->dtype);
        if (small) {
            if (!o->states32[i]) {
                std::unique_ptr<State32> s(new State32());
                int rc = s->allocate(p->numel);
                if (rc) return rc;
                o->states32[i] = std::move(s);
            }
            EriAdamW32Tensor r;
            std::memset(&r, 0, sizeof r);
            r.p = p->data;
            r.g = p->grad;
            r.m = o->states32[i]->m;
            r.v = o->states32[i]->v;
            r.numel = p->numel;
            r.dtype_tag = p->dtype;
            r.grad_scale = o->param_scale[i];
            scaled = scaled || o->param_scale[i] != 1.0f;
            rows32.push_back(r);
            continue;
        }
        if (!o->states[i]) { // init_state :179-199
            std::unique_ptr<State8> s(new State8());
            int rc = s->allocate(p->numel, o->stream, o->state_pool, o->state_lane);
            if (rc) return rc;
            o->states[i] = std::move(s);
        }
        State8 &s = *o->states[i];
        EriAdam8Tensor r;
        std::memset(&r, 0, sizeof r);
        r.p = p->data;
        r.g = p->grad;
        r.m = s.m;
        r.v = s.v;
        r.absmax_m = s.absmax_m;
        r.absmax_v = s.absmax_v;
        r.numel = p->numel;
        r.block_start = start;
        r.dtype_tag = p->dtype;
        r.grad_f32 = (p->dtype == ERI_DTYPE_BF16 && p->grad_dtype == ERI_DTYPE_F32) ? 1 : 0;
        r.grad_scale = o->param_scale[i];
        scaled = scaled || o->param_scale[i] != 1.0f;
        start += blocks_of(p->numel);
        ids.push_back(i);
        rows.push_back(r);
    }
    if (skipped) *skipped = skip;
    const bool clip = o->max_grad_norm > 0.0f;
    // Attached EMA model: EMAModel::update (ema_enhanced.rs:79-104) as part of this step.  Parameters that
    // take the 8-bit step carry their shadow in their row (the step updates it, inside the kernel where
    // that pays); the others -- no gradient this step, fp32 moments -- get the plain sweep afterwards, and
    // a name seen for the first time gets a copy of its parameter as the reference does (:100-103).
    float ema_decay = 0.0f;
    std::vector<EriEmaTensor> ema_others;
    std::vector<uint32_t> ema_new;
    bool ema_rows = false;
    if (o->ema) {
        o->ema->step += 1;                       // :80
        ema_decay = eri_ema_current_decay(o->ema); // :83
        size_t k = 0;
        for (uint32_t i = 0; i < o->params.size(); ++i) {
            const EriParameter *p = o->params[i];
            const bool in_table = k < ids.size() && ids[k] == i;
            auto it = o->ema->shadows.find(o->ema_names[i]);
            if (it == o->ema->shadows.end() || it->second.numel != p->numel || it->second.dtype != p->dtype) {
                ema_new.push_back(i);
            } else if (in_table) {
                rows[k].ema_shadow = it->second.data;
                ema_rows = true;
            } else {
                EriEmaTensor r;
                r.shadow = it->second.data;
                r.p = p->data;
                r.numel = p->numel;
                r.dtype_tag = p->dtype;
                r.reserved = 0;
                ema_others.push_back(r);
            }
            if (in_table) ++k;
        }
    }
    if (!rows32.empty() && o->mode != ERI_ADAM8_MODE_ERI) // refused before anything is launched
        return fail(ERI_ERR_ARG, "InvalidOperation: min_8bit_size needs mode ERI");
    // Everything that can be refused comes before the first launch: both launch tables are built or refreshed
    // here, so that a step that fails on them has changed nothing.
    int rc = 0;
    if (!rows.empty()) {
        if (!o->table || ids != o->table_ids) {
            if (o->table) eri_adam8_table_destroy(o->table);
            o->table = nullptr;
            o->norm_table = nullptr; // whichever table held the last norm, its result may have lived in this one
            rc = eri_adam8_table_create(rows.data(), (uint32_t)rows.size(), o->stream, &o->table);
            if (rc) return rc;
            o->table_ids = ids;
            o->table_rows = rows;
            o->have_qerr = false;
        } else if (std::memcmp(rows.data(), o->table_rows.data(), rows.size() * sizeof(EriAdam8Tensor)) != 0) {
            rc = eri_adam8_table_update(o->table, rows.data(), (uint32_t)rows.size(), o->stream);
            if (rc) return rc;
            o->table_rows = rows;
        }
    }
    // The tensors kept in 32-bit moments are clipped by the same global norm as the rest
    // (pipeline_flux_lora_1024.rs:691-697 clips every trainable gradient, then steps): their gradients go into
    // a gradient-only table that is normed together with the 8-bit table.
    if (clip && !rows32.empty()) {
        std::vector<EriAdam8Tensor> grows(rows32.size());
        uint64_t gstart = 0;
        for (size_t k = 0; k < rows32.size(); ++k) {
            EriAdam8Tensor &g = grows[k];
            std::memset(&g, 0, sizeof g);
            g.p = rows32[k].p;
            g.g = rows32[k].g;
            g.numel = rows32[k].numel;
            g.dtype_tag = rows32[k].dtype_tag;
            g.block_start = gstart;
            g.grad_scale = 1.0f;
            gstart += blocks_of(g.numel);
        }
        bool same = o->grad_table && o->grad_rows.size() == grows.size();
        for (size_t k = 0; same && k < grows.size(); ++k)
            same = grows[k].numel == o->grad_rows[k].numel && grows[k].dtype_tag == o->grad_rows[k].dtype_tag;
        if (!same) {
            if (o->grad_table) eri_adam8_table_destroy(o->grad_table);
            o->grad_table = nullptr;
            o->norm_table = nullptr;
            o->grad_rows.clear();
            rc = eri_adam8_grad_table_create(grows.data(), (uint32_t)grows.size(), o->stream, &o->grad_table);
            if (rc) return rc;
            o->grad_rows = grows;
        } else if (std::memcmp(grows.data(), o->grad_rows.data(), grows.size() * sizeof(EriAdam8Tensor)) != 0) {
            rc = eri_adam8_table_update(o->grad_table, grows.data(), (uint32_t)grows.size(), o->stream);
            if (rc) return rc;
            o->grad_rows = grows;
        }
    }
    if (clip) { // one norm over every gradient of this step
        if (!rows.empty() && !rows32.empty())
            rc = eri_adam8_grad_norm_joint(o->table, o->grad_table, o->max_grad_norm, o->clip_denom_eps, o->stream);
        else
            rc = eri_adam8_grad_norm(rows.empty() ? o->grad_table : o->table, o->max_grad_norm, o->clip_denom_eps, o->stream);
        if (rc) return rc;
        o->norm_table = rows.empty() ? o->grad_table : o->table;
    }
    if (!rows32.empty()) {
        // The reference's update with fp32 moments: the 32-bit step computes
        // p + ((m/(sqrt(v)+eps)) + p*wd) * (-lr), which with lr = the bias-corrected step size is
        // adam8bit_enhanced.rs:252-275 bit for bit (x * (-a) = -(x * a), p + (-y) = p - y).
        EriAdam8Hyper h8;
        rc = eri_adam8_hyper_pack(o->lr, o->beta1, o->beta2, o->eps, o->wd, o->step, ERI_ADAM8_MODE_ERI, 0, &h8);
        if (rc) return rc;
        EriAdamW32Hyper h32;
        h32.lr = h8.step_size;
        h32.beta1 = h8.beta1;
        h32.beta2 = h8.beta2;
        h32.eps = h8.eps;
        h32.weight_decay = h8.weight_decay > 0.0f ? h8.weight_decay : 0.0f; // :267: decay only if positive
        if (scaled || clip) { // the factors the 8-bit rows get inside their kernel, in the same order
            const float *dev_scale = nullptr;
            if (clip) {
                rc = eri_adam8_grad_norm_scale_ptr(o->norm_table, &dev_scale);
                if (rc) return rc;
            }
            rc = eri_adamw32_step_multi_scaled(rows32.data(), (uint32_t)rows32.size(), &h32, o->grad_scale, dev_scale, o->stream);
        } else {
            rc = eri_adamw32_step_multi(rows32.data(), (uint32_t)rows32.size(), &h32, o->stream);
        }
        if (rc) return rc;
    }
    if (rows.empty()) return adam8bit_ema_rest(o, ema_others, ema_new, ema_decay);
    EriAdam8Hyper h;
    uint32_t flags = o->flags | ((scaled || clip) ? (uint32_t)ERI_ADAM8_FLAG_GRAD_SCALE : 0u) |
                     (clip ? (uint32_t)ERI_ADAM8_FLAG_CLIP_FROM_TABLE : 0u);
    rc = eri_adam8_hyper_pack(o->lr, o->beta1, o->beta2, o->eps, o->wd, o->step, o->mode, flags, &h);
    if (rc) return rc;
    h.grad_scale = o->grad_scale;
    if (o->track_qerr) {
        EriAdam8Hyper hq = h; // the moments of mode BNB are those of mode ERI; the statistics pass knows ERI
        if (o->mode == ERI_ADAM8_MODE_BNB) {
            rc = eri_adam8_hyper_pack(o->lr, o->beta1, o->beta2, o->eps, o->wd, o->step, ERI_ADAM8_MODE_ERI, flags, &hq);
            if (rc) return rc;
            hq.grad_scale = o->grad_scale;
        }
        rc = eri_adam8_quant_error(o->table, &hq, o->stream);
        if (rc) return rc;
        o->have_qerr = true;
    }
    if (ema_rows) {
        h.flags |= ERI_ADAM8_FLAG_EMA;
        h.ema_decay = ema_decay;
    }
    rc = eri_adam8_step_table(o->table, &h, o->stream);
    if (rc) return rc;
    return adam8bit_ema_rest(o, ema_others, ema_new, ema_decay);
}

int eri_adam8bit_zero_grad(EriAdam8bit *o) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    for (auto *p : o->params) p->grad = nullptr;
    return 0;
}

double eri_adam8bit_current_lr(const EriAdam8bit *o) { return o ? o->lr : 0.0; }

int eri_adam8bit_set_learning_rate(EriAdam8bit *o, double lr) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->lr = lr;
    return 0;
}

uint64_t eri_adam8bit_quantized_memory_usage(const EriAdam8bit *o) {
    uint64_t total = 0;
    if (o)
    {
        for (auto &s : o->states)
            if (s) total += s->nbytes();
        for (auto &s : o->states32)
            if (s) total += s->nbytes();
    }
    return total;
}

uint64_t eri_adam8bit_get_step(const EriAdam8bit *o) { return o ? o->step : 0; }

int eri_adam8bit_set_grad_scale(EriAdam8bit *o, float scale) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->grad_scale = scale;
    return 0;
}

int eri_adam8bit_set_param_grad_scale(EriAdam8bit *o, uint32_t index, float scale) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (index >= o->param_scale.size()) return fail(ERI_ERR_ARG, "parameter index out of range");
    o->param_scale[index] = scale;
    return 0;
}

int eri_adam8bit_set_max_grad_norm(EriAdam8bit *o, float max_norm, float denom_eps) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->max_grad_norm = max_norm;
    o->clip_denom_eps = denom_eps;
    return 0;
}

int eri_adam8bit_last_grad_norm(EriAdam8bit *o, float *norm, float *scale) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (!o->norm_table) return fail(ERI_ERR_ARG, "no step with gradient clipping has run yet");
    return eri_adam8_grad_norm_read(o->norm_table, norm, scale, o->stream);
}

int eri_adam8bit_last_nonfinite_grads(EriAdam8bit *o, uint64_t *count) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (!o->norm_table) return fail(ERI_ERR_ARG, "no step with gradient clipping has run yet");
    return eri_adam8_grad_nonfinite_read(o->norm_table, count, o->stream);
}

int eri_adam8bit_track_quantization_error(EriAdam8bit *o, int enabled) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->track_qerr = enabled != 0;
    return 0;
}

int eri_adam8bit_quantization_stats(EriAdam8bit *o, float *m_error, float *v_error) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (!o->have_qerr || !o->table) { // nothing tracked yet: the reference reports 0 for an empty map (:320)
        if (m_error) *m_error = 0.0f;
        if (v_error) *v_error = 0.0f;
        return 0;
    }
    return eri_adam8_quant_error_read(o->table, m_error, v_error, o->stream);
}

int eri_adam8bit_set_mode(EriAdam8bit *o, int mode) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (mode != ERI_ADAM8_MODE_ERI && mode != ERI_ADAM8_MODE_BNB)
        return fail(ERI_ERR_ARG, "the list-of-parameters optimizer steps in mode ERI or BNB");
    o->mode = mode;
    return 0;
}

int eri_adam8bit_attach_ema(EriAdam8bit *o, EriEmaModel *ema, const char *const *names, uint32_t n) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (!ema) { // detach
        o->ema = nullptr;
        o->ema_names.clear();
        return 0;
    }
    if (!names) return fail(ERI_ERR_NULL, "names is NULL");
    if (n != o->params.size()) return fail(ERI_ERR_ARG, "attach_ema: one name per parameter of the optimizer");
    if (ema->stream != o->stream) return fail(ERI_ERR_ARG, "attach_ema: the EMA model and the optimizer must use the same stream");
    std::vector<std::string> v;
    for (uint32_t i = 0; i < n; ++i) {
        if (!names[i]) return fail(ERI_ERR_NULL, "a name is NULL");
        v.emplace_back(names[i]);
    }
    o->ema = ema;
    o->ema_names.swap(v);
    return 0;
}

int eri_adam8bit_set_state_pool(EriAdam8bit *o, EriHipPool *pool, uint32_t lane) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->state_pool = pool;
    o->state_lane = lane;
    return 0;
}

int eri_adam8bit_set_min_8bit_size(EriAdam8bit *o, uint64_t numel) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->min_8bit_size = numel;
    return 0;
}

int eri_adam8bit_state32_ptrs(const EriAdam8bit *o, uint32_t index, float **m, float **v) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (index >= o->states32.size()) return fail(ERI_ERR_ARG, "parameter index out of range");
    const State32 *s = o->states32[index].get();
    if (m) *m = s ? s->m : nullptr;
    if (v) *v = s ? s->v : nullptr;
    return 0;
}

int eri_adam8bit_set_flags(EriAdam8bit *o, uint32_t flags) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->flags = flags;
    return 0;
}

int eri_adam8bit_state_ptrs(const EriAdam8bit *o, uint32_t index, uint8_t **m, uint8_t **v, float **absmax_m,
                            float **absmax_v) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (index >= o->states.size()) return fail(ERI_ERR_ARG, "parameter index out of range");
    const State8 *s = o->states[index].get();
    if (m) *m = s ? s->m : nullptr;
    if (v) *v = s ? s->v : nullptr;
    if (absmax_m) *absmax_m = s ? s->absmax_m : nullptr;
    if (absmax_v) *absmax_v = s ? s->absmax_v : nullptr;
    return 0;
}

int eri_adam8bit_save_state(EriAdam8bit *o, const char *path) {
    if (!o || !path) return fail(ERI_ERR_NULL, "optimizer or path is NULL");
    // header from the sizes alone, then every state streamed behind it through pinned memory
    StWriter w;
    char buf[64];
    std::map<std::string, std::string> meta;
    meta["format"] = "eri-adam8bit-blockwise-v1";
    meta["block_size"] = "2048";
    std::snprintf(buf, sizeof buf, "%llu", (unsigned long long)o->step);
    meta["step"] = buf;
    std::snprintf(buf, sizeof buf, "%.17g", o->lr);
    meta["learning_rate"] = buf;
    w.begin(meta);
    bool any = false;
    for (uint32_t i = 0; i < o->states.size(); ++i) {
        const State8 *s = o->states[i].get();
        if (!s) continue;
        any = true;
        const uint64_t nb = blocks_of(s->numel);
        const std::string base = "optimizer.param_" + std::to_string(i);
        w.add(base + ".m", "U8", s->numel, s->numel);
        w.add(base + ".v", "U8", s->numel, s->numel);
        w.add(base + ".absmax_m", "F32", nb, nb * 4);
        w.add(base + ".absmax_v", "F32", nb, nb * 4);
    }
    for (uint32_t i = 0; i < o->states32.size(); ++i) { // fp32 moments of the parameters below min_8bit_size
        const State32 *s = o->states32[i].get();
        if (!s) continue;
        any = true;
        const std::string base = "optimizer.param_" + std::to_string(i);
        w.add(base + ".m32", "F32", s->numel, s->numel * 4);
        w.add(base + ".v32", "F32", s->numel, s->numel * 4);
    }
    Bounce bounce;
    if (any) {
        int rc = bounce.ensure();
        if (rc) return rc;
    }
    std::ofstream f(path, std::ios::binary | std::ios::trunc);
    if (!f || !w.write_header(f))
        return fail(ERI_ERR_ARG, std::string("InvalidOperation: Failed to save optimizer: cannot write ") + path);
    for (uint32_t i = 0; i < o->states.size(); ++i) {
        const State8 *s = o->states[i].get();
        if (!s) continue;
        const uint64_t nb = blocks_of(s->numel);
        const uint64_t sizes[4] = {s->numel, s->numel, nb * 4, nb * 4};
        const void *src[4] = {s->m, s->v, s->absmax_m, s->absmax_v};
        for (int k = 0; k < 4; ++k) {
            int rc = stream_out(f, src[k], sizes[k], bounce, o->stream);
            if (rc) return rc;
        }
    }
    for (uint32_t i = 0; i < o->states32.size(); ++i) {
        const State32 *s = o->states32[i].get();
        if (!s) continue;
        int rc = stream_out(f, s->m, s->numel * 4, bounce, o->stream);
        if (!rc) rc = stream_out(f, s->v, s->numel * 4, bounce, o->stream);
        if (rc) return rc;
    }
    f.flush();
    if (!f) return fail(ERI_ERR_ARG, std::string("InvalidOperation: Failed to save optimizer: cannot write ") + path);
    return 0;
}

int eri_adam8bit_load_state(EriAdam8bit *o, const char *path) {
    if (!o || !path) return fail(ERI_ERR_NULL, "optimizer or path is NULL");
    std::ifstream f(path, std::ios::binary);
    if (!f) return fail(ERI_ERR_ARG, std::string("InvalidOperation: Failed to read optimizer: cannot open ") + path);
    StFile st;
    std::string why;
    if (!parse_safetensors(f, st, why))
        return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: " + why);
    if (!st.metadata.count("step") || !st.metadata.count("learning_rate"))
        return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: step / learning_rate missing");
    // validate everything before touching the optimizer
    struct Item { uint32_t idx; const StEntry *e[4]; };
    std::vector<Item> items, items32;
    for (uint32_t i = 0; i < o->params.size(); ++i) {
        const std::string base = "optimizer.param_" + std::to_string(i);
        auto m32 = st.tensors.find(base + ".m32");
        if (m32 != st.tensors.end()) { // fp32 moments
            auto v32 = st.tensors.find(base + ".v32");
            const uint64_t bytes = o->params[i]->numel * 4;
            if (v32 == st.tensors.end() || m32->second.dtype != "F32" || v32->second.dtype != "F32" ||
                m32->second.end - m32->second.begin != bytes || v32->second.end - v32->second.begin != bytes)
                return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: size or dtype mismatch for " + base);
            items32.push_back({i, {&m32->second, &v32->second, nullptr, nullptr}});
            continue;
        }
        auto m = st.tensors.find(base + ".m");
        if (m == st.tensors.end()) continue;
        auto v = st.tensors.find(base + ".v"), am = st.tensors.find(base + ".absmax_m"), av = st.tensors.find(base + ".absmax_v");
        if (v == st.tensors.end() || am == st.tensors.end() || av == st.tensors.end())
            return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: incomplete state for " + base);
        const uint64_t n = o->params[i]->numel, nb = blocks_of(n);
        const StEntry *e[4] = {&m->second, &v->second, &am->second, &av->second};
        const uint64_t want[4] = {n, n, nb * 4, nb * 4};
        const char *dt[4] = {"U8", "U8", "F32", "F32"};
        for (int k = 0; k < 4; ++k)
            if (e[k]->end - e[k]->begin != want[k] || e[k]->dtype != dt[k])
                return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: size or dtype mismatch for " + base);
        items.push_back({i, {e[0], e[1], e[2], e[3]}});
    }
    // the new states are complete before the first one replaces an old one: a failure half way
    // through the file leaves the optimizer as it was
    Bounce bounce;
    std::vector<std::unique_ptr<State8>> fresh;
    for (auto &it : items) {
        int rc = bounce.ensure();
        if (rc) return rc;
        std::unique_ptr<State8> s(new State8());
        rc = s->allocate(o->params[it.idx]->numel, o->stream, o->state_pool, o->state_lane);
        if (rc) return rc;
        void *dst[4] = {s->m, s->v, s->absmax_m, s->absmax_v};
        for (int k = 0; k < 4; ++k) {
            rc = stream_in(f, st.data_start + it.e[k]->begin, dst[k], it.e[k]->end - it.e[k]->begin, bounce, o->stream);
            if (rc) return rc;
        }
        fresh.push_back(std::move(s));
    }
    std::vector<std::unique_ptr<State32>> fresh32;
    for (auto &it : items32) {
        int rc = bounce.ensure();
        if (rc) return rc;
        std::unique_ptr<State32> s(new State32());
        rc = s->allocate(o->params[it.idx]->numel);
        if (rc) return rc;
        void *dst[2] = {s->m, s->v};
        for (int k = 0; k < 2; ++k) {
            rc = stream_in(f, st.data_start + it.e[k]->begin, dst[k], it.e[k]->end - it.e[k]->begin, bounce, o->stream);
            if (rc) return rc;
        }
        fresh32.push_back(std::move(s));
    }
    for (size_t k = 0; k < items.size(); ++k) {
        o->states[items[k].idx] = std::move(fresh[k]);
        o->states32[items[k].idx].reset();
    }
    for (size_t k = 0; k < items32.size(); ++k) {
        o->states32[items32[k].idx] = std::move(fresh32[k]);
        o->states[items32[k].idx].reset();
    }
    o->step = std::strtoull(st.metadata["step"].c_str(), nullptr, 10);
    o->lr = std::strtod(st.metadata["learning_rate"].c_str(), nullptr);
    if (o->table) { // state pointers changed
        eri_adam8_table_destroy(o->table);
        o->table = nullptr;
        o->norm_table = nullptr;
        o->table_ids.clear();
    }
    return 0;
}

namespace {

/* Cursor over a bincode 1.x (default options) byte stream. */
struct Bincode {
    const unsigned char *p, *e;
    bool ok = true;
    bool need(size_t n) {
        if ((size_t)(e - p) < n) ok = false;
        return ok;
    }
    uint64_t u64() {
        uint64_t v = 0;
        if (need(8)) { std::memcpy(&v, p, 8); p += 8; }
        return v;
    }
    float f32() {
        float v = 0;
        if (need(4)) { std::memcpy(&v, p, 4); p += 4; }
        return v;
    }
    double f64() {
        double v = 0;
        if (need(8)) { std::memcpy(&v, p, 8); p += 8; }
        return v;
    }
    int8_t i8() {
        int8_t v = 0;
        if (need(1)) { v = (int8_t)*p; p += 1; }
        return v;
    }
};

/* One QuantizedTensor of the file, left where it lies in the mapped file. */
struct LegacyTensor {
    const int8_t *q = nullptr;
    uint64_t n = 0;
    float scale = 1.0f;
    int8_t zp = 0;
};

/* A file mapped read-only: a state file of a large model is walked in place, never copied whole. */
struct MappedFile {
    const unsigned char *data = nullptr;
    size_t size = 0;
    bool open(const char *path) {
        const int fd = ::open(path, O_RDONLY);
        if (fd < 0) return false;
        struct stat st;
        if (::fstat(fd, &st) != 0 || !S_ISREG(st.st_mode)) {
            ::close(fd);
            return false;
        }
        size = (size_t)st.st_size;
        if (size) {
            void *m = ::mmap(nullptr, size, PROT_READ, MAP_PRIVATE, fd, 0);
            if (m == MAP_FAILED) {
                ::close(fd);
                size = 0;
                return false;
            }
            data = static_cast<const unsigned char *>(m);
        }
        ::close(fd);
        return true;
    }
    ~MappedFile() {
        if (data) ::munmap(const_cast<unsigned char *>(data), size);
    }
};

bool read_legacy_map(Bincode &b, std::map<std::string, LegacyTensor> &out) {
    const uint64_t count = b.u64();
    if (!b.ok || count > (1u << 24)) return false;
    for (uint64_t k = 0; k < count; ++k) {
        const uint64_t klen = b.u64();
        if (!b.ok || klen > 4096 || !b.need(klen)) return false;
        std::string key(reinterpret_cast<const char *>(b.p), (size_t)klen);
        b.p += klen;
        const uint64_t n = b.u64();
        if (!b.ok || !b.need(n)) return false;
        const int8_t *q = reinterpret_cast<const int8_t *>(b.p);
        b.p += n;
        const float scale = b.f32();
        const int8_t zp = b.i8();
        const uint64_t rank = b.u64();
        if (!b.ok || rank > 16) return false;
        for (uint64_t d = 0; d < rank; ++d) b.u64();
        b.f32(); // quantization_error
        if (!b.ok) return false;
        LegacyTensor t;
        t.q = q;
        t.n = n;
        t.scale = scale;
        t.zp = zp;
        out[key] = t;
    }
    return true;
}

} // namespace

extern "C" int eri_adam8bit_load_legacy_state(EriAdam8bit *o, const char *path) {
    if (!o || !path) return fail(ERI_ERR_NULL, "optimizer or path is NULL");
    MappedFile raw;
    if (!raw.open(path)) return fail(ERI_ERR_ARG, std::string("InvalidOperation: Failed to read optimizer: cannot open ") + path);
    Bincode b{raw.data, raw.data + raw.size};
    const uint64_t step = b.u64();
    std::map<std::string, LegacyTensor> first, second;
    if (!read_legacy_map(b, first) || !read_legacy_map(b, second))
        return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: truncated or malformed bincode");
    const double lr = b.f64();
    if (!b.ok || b.p != b.e)
        return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: trailing or missing bytes");
    struct Item { uint32_t idx; const LegacyTensor *m, *v; };
    std::vector<Item> items;
    for (uint32_t i = 0; i < o->params.size(); ++i) {
        const std::string key = "param_" + std::to_string(i);
        auto m = first.find(key), v = second.find(key);
        if (m == first.end() && v == second.end()) continue;
        if (m == first.end() || v == second.end() || m->second.n != o->params[i]->numel ||
            v->second.n != o->params[i]->numel)
            return fail(ERI_ERR_ARG, "InvalidOperation: Failed to deserialize optimizer: state of " + key + " does not fit its parameter");
        items.push_back({i, &m->second, &v->second});
    }
    // dequantised as the reference does (to_tensor, adam8bit_enhanced.rs:117-129) piece by piece into
    // pinned memory, gathered in one fp32 device buffer per tensor, quantised blockwise from there;
    // every new state is complete before the first one replaces an old one
    uint64_t largest = 0;
    for (auto &it : items) largest = std::max<uint64_t>(largest, o->params[it.idx]->numel);
    void *tmp = nullptr;
    Bounce bounce;
    if (!items.empty()) {
        int dev = 0;
        int rc = eri_hip_get_device(&dev);
        if (!rc) rc = bounce.ensure();
        if (!rc) rc = eri_hip_malloc_zeroed(dev, largest * 4, &tmp);
        if (rc) return rc;
    }
    std::vector<std::unique_ptr<State8>> fresh;
    int rc = 0;
    for (auto &it : items) {
        const uint64_t n = o->params[it.idx]->numel;
        std::unique_ptr<State8> s(new State8());
        rc = s->allocate(n, o->stream, o->state_pool, o->state_lane);
        for (int k = 0; k < 2 && rc == 0; ++k) {
            const LegacyTensor *src = k == 0 ? it.m : it.v;
            const uint64_t piece = Bounce::kHalf / 4;
            for (uint64_t done = 0; done < n && rc == 0; done += piece) {
                const uint64_t cnt = n - done < piece ? n - done : piece;
                float *buf = reinterpret_cast<float *>(bounce.next());
                for (uint64_t i = 0; i < cnt; ++i) {
                    const float x = ((float)src->q[done + i] - (float)src->zp) * src->scale;
                    buf[i] = std::isfinite(x) ? x : 0.0f;
                }
                rc = eri_hip_stream_sync(o->stream); // the copy out of the other half
                if (rc == 0) rc = eri_hip_memcpy_async(static_cast<float *>(tmp) + done, buf, cnt * 4, 1, o->stream);
            }
            if (rc == 0)
                rc = eri_adam8_quantize(static_cast<const float *>(tmp), k == 0 ? 1 : 0, n, k == 0 ? s->m : s->v,
                                        k == 0 ? s->absmax_m : s->absmax_v, o->stream);
            if (rc == 0) rc = eri_hip_stream_sync(o->stream);
        }
        if (rc) break;
        fresh.push_back(std::move(s));
    }
    if (tmp) eri_hip_free(tmp);
    if (rc) return rc;
    for (size_t k = 0; k < items.size(); ++k) o->states[items[k].idx] = std::move(fresh[k]);
    o->step = step;
    o->lr = lr;
    if (o->table) {
        eri_adam8_table_destroy(o->table);
        o->table = nullptr;
        o->norm_table = nullptr;
        o->table_ids.clear();
    }
    return 0;
}

// ---- functional flavour ------------------------------------------------------------------------

int eri_adam8bit_fn_with_params(double lr, double beta1, double beta2, double eps, double weight_decay, void *stream,
                                EriAdam8bitFn **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    EriAdam8bitFn *o = new EriAdam8bitFn();
    o->lr = lr;
    o->beta1 = beta1;
    o->beta2 = beta2;
    o->eps = eps;
    o->wd = weight_decay;
    o->stream = stream;
    *out = o;
    return 0;
}

int eri_adam8bit_fn_destroy(EriAdam8bitFn *o) {
    if (!o) return 0;
    int rc = fn_flush(o); // an update that was accepted runs
    delete o;
    return rc;
}

} // extern "C"

namespace {

/* The state of `name`, created on first use (adam8bit.rs:126-130).  `hint` is the position of this update in
 * the batch: trainers update the same names in the same order every step, so the name usually matches the
 * one the last flush had at that position and the map is not searched. */
int fn_state_of(EriAdam8bitFn *o, const char *name, uint64_t numel, size_t hint, const std::string **key, FnState **out) {
    if (hint < o->last_order.size() && *o->last_order[hint].first == name) {
        *key = o->last_order[hint].first;
        *out = o->last_order[hint].second;
    } else {
        auto it = o->states.find(std::string_view(name));
        if (it == o->states.end()) {
            std::unique_ptr<FnState> s(new FnState());
            int rc = s->allocate(numel, o->stream, o->state_pool, o->state_lane);
            if (rc) return rc;
            it = o->states.emplace(name, std::move(s)).first;
        }
        *key = &it->first;
        *out = it->second.get();
    }
    if ((*out)->numel != numel) return fail(ERI_ERR_ARG, std::string("state of '") + name + "' has a different size");
    return 0;
}

int fn_check_update(const char *name, const void *param, const void *grad, uint64_t numel, int dtype_tag,
                    int grad_dtype_tag, const void *out) {
    if (!name || !param || !grad || !out) return fail(ERI_ERR_NULL, "update with NULL argument");
    if (numel == 0) return fail(ERI_ERR_EMPTY, "InvalidOperation: Empty tensor for quantization");
    if (dtype_tag != ERI_DTYPE_F32 && dtype_tag != ERI_DTYPE_BF16)
        return fail(ERI_ERR_DTYPE, "Unsupported: 8-bit Adam takes F32 or BF16 parameters");
    if (grad_dtype_tag != dtype_tag && !(dtype_tag == ERI_DTYPE_BF16 && grad_dtype_tag == ERI_DTYPE_F32))
        return fail(ERI_ERR_DTYPE, "Unsupported: a gradient has the dtype of its parameter, or F32 for a BF16 parameter");
    if (((uintptr_t)param | (uintptr_t)grad | (uintptr_t)out) & 15u)
        return fail(ERI_ERR_ALIGN, "update: param, grad and out must be 16-byte aligned");
    return 0;
}

EriAdam8Tensor fn_row(const FnState &s, const void *param, const void *grad, uint64_t numel, int dtype_tag,
                      int grad_dtype_tag, void *out) {
    EriAdam8Tensor r;
    std::memset(&r, 0, sizeof r);
    r.p = out;
    r.p_src = out == param ? nullptr : param; // the kernel reads the old values from param and writes out: no copy
    r.g = grad;
    r.m = s.m;
    r.v = s.v;
    r.absmax_m = s.absmax_m;
    r.absmax_v = s.absmax_v;
    r.numel = numel;
    r.block_start = 0;
    r.dtype_tag = dtype_tag;
    r.grad_f32 = (dtype_tag == ERI_DTYPE_BF16 && grad_dtype_tag == ERI_DTYPE_F32) ? 1 : 0;
    r.grad_scale = 1.0f;
    return r;
}

int fn_hyper(const EriAdam8bitFn *o, EriAdam8Hyper *h) {
    // the bias correction uses the counter as it stands; step() bumps it later (:107,:164)
    return eri_adam8_hyper_pack(o->lr, o->beta1, o->beta2, o->eps, o->wd, o->step, ERI_ADAM8_MODE_L2,
                                ERI_ADAM8_FLAG_EXACT_PARAM, h);
}

/* One launch over every queued row.  The launch tables of the last two distinct row sets are kept: rows that
 * equal one of them cost nothing, the same tensors with new pointers cost one small upload into the table
 * that was used longer ago. */
int fn_flush(EriAdam8bitFn *o) {
    if (o->pending.empty()) return 0;
    std::vector<EriAdam8Tensor> rows;
    rows.swap(o->pending);
    std::vector<std::pair<const std::string *, FnState *>> who;
    who.swap(o->pending_who);
    o->generation += 1;
    uint64_t start = 0;
    for (auto &r : rows) {
        r.block_start = start;
        start += blocks_of(r.numel);
    }
    EriAdam8Hyper h;
    int rc = fn_hyper(o, &h);
    if (rc) return rc;
    o->flushes += 1;
    const size_t bytes = rows.size() * sizeof(EriAdam8Tensor);
    // the table used longer ago first: that is the one an alternating trainer comes back to
    const int older = o->slots[0].used <= o->slots[1].used ? 0 : 1;
    EriAdam8bitFn::TableSlot *hit = nullptr;
    for (int k : {older, 1 - older}) {
        auto &sl = o->slots[k];
        if (sl.table && sl.rows.size() == rows.size() && std::memcmp(rows.data(), sl.rows.data(), bytes) == 0) {
            hit = &sl;
            break;
        }
    }
    if (!hit) {
        auto &sl = o->slots[older];
        bool same = sl.table && sl.rows.size() == rows.size();
        for (size_t i = 0; same && i < rows.size(); ++i)
            same = rows[i].numel == sl.rows[i].numel && rows[i].dtype_tag == sl.rows[i].dtype_tag &&
                   rows[i].grad_f32 == sl.rows[i].grad_f32;
        if (!same) {
            if (sl.table) eri_adam8_table_destroy(sl.table);
            sl.table = nullptr;
            sl.rows.clear();
            rc = eri_adam8_table_create(rows.data(), (uint32_t)rows.size(), o->stream, &sl.table);
        } else {
            rc = eri_adam8_table_update(sl.table, rows.data(), (uint32_t)rows.size(), o->stream);
        }
        if (rc) {
            sl.rows.clear(); // whatever the table holds now, it is not a set to come back to
            return rc;
        }
        sl.rows.swap(rows);
        o->uploads += 1;
        hit = &sl;
    }
    hit->used = o->flushes;
    o->last_order.swap(who);
    return eri_adam8_step_table(hit->table, &h, o->stream);
}

int fn_enqueue(EriAdam8bitFn *o, const char *name, const void *param, const void *grad, uint64_t numel, int dtype_tag,
               int grad_dtype_tag, void *out) {
    int rc = fn_check_update(name, param, grad, numel, dtype_tag, grad_dtype_tag, out);
    if (rc) return rc;
    const std::string *key = nullptr;
    FnState *s = nullptr;
    rc = fn_state_of(o, name, numel, o->pending.size(), &key, &s);
    if (rc) return rc;
    if (s->queued_in == o->generation) { // the same name twice in one batch: the first update must run first
        rc = fn_flush(o);
        if (rc) return rc;
    }
    s->queued_in = o->generation;
    o->pending.push_back(fn_row(*s, param, grad, numel, dtype_tag, grad_dtype_tag, out));
    o->pending_who.emplace_back(key, s);
    return 0;
}

} // namespace

extern "C" {

int eri_adam8bit_fn_update(EriAdam8bitFn *o, const char *name, const void *param, const void *grad, uint64_t numel,
                           int dtype_tag, int grad_dtype_tag, void *out) {
    if (!o) return fail(ERI_ERR_NULL, "update with NULL argument");
    if (o->batching) return fn_enqueue(o, name, param, grad, numel, dtype_tag, grad_dtype_tag, out);
    // immediate: one launch per call through the state's own one-row table
    int rc = fn_check_update(name, param, grad, numel, dtype_tag, grad_dtype_tag, out);
    if (rc) return rc;
    const std::string *key = nullptr;
    FnState *sp = nullptr;
    rc = fn_state_of(o, name, numel, o->last_order.size(), &key, &sp);
    if (rc) return rc;
    FnState &s = *sp;
    const EriAdam8Tensor r = fn_row(s, param, grad, numel, dtype_tag, grad_dtype_tag, out);
    EriAdam8Hyper h;
    rc = fn_hyper(o, &h);
    if (rc) return rc;
    if (!s.table) {
        rc = eri_adam8_table_create(&r, 1, o->stream, &s.table);
        if (rc) return rc;
        s.row = r;
    } else if (std::memcmp(&r, &s.row, sizeof r) != 0) { // same size by the check above; new pointers or dtype
        if (r.dtype_tag != s.row.dtype_tag || r.grad_f32 != s.row.grad_f32) {
            eri_adam8_table_destroy(s.table);
            s.table = nullptr;
            rc = eri_adam8_table_create(&r, 1, o->stream, &s.table);
        } else {
            rc = eri_adam8_table_update(s.table, &r, 1, o->stream);
        }
        if (rc) return rc;
        s.row = r;
    }
    return eri_adam8_step_table(s.table, &h, o->stream);
}

int eri_adam8bit_fn_update_many(EriAdam8bitFn *o, const char *const *names, const void *const *params,
                                const void *const *grads, const uint64_t *numels, const int32_t *dtype_tags,
                                const int32_t *grad_dtype_tags, void *const *outs, uint32_t n) {
    if (!o || !names || !params || !grads || !numels || !dtype_tags || !outs)
        return fail(ERI_ERR_NULL, "update_many with NULL argument");
    // 1. every row is checked before anything runs: arguments, and the size of a state that exists already.
    //    Trainers update the same names in the same order every step, so the name at position i is usually the
    //    one the last flush had there and the map is not searched.
    std::vector<uint32_t> unknown;
    for (uint32_t i = 0; i < n; ++i) {
        int rc = fn_check_update(names[i], params[i], grads[i], numels[i], dtype_tags[i],
                                 grad_dtype_tags ? grad_dtype_tags[i] : dtype_tags[i], outs[i]);
        if (rc) return rc;
        const FnState *known = nullptr;
        if (i < o->last_order.size() && *o->last_order[i].first == names[i]) {
            known = o->last_order[i].second;
        } else {
            auto it = o->states.find(std::string_view(names[i]));
            if (it != o->states.end()) known = it->second.get();
        }
        if (!known) unknown.push_back(i);
        else if (known->numel != numels[i])
            return fail(ERI_ERR_ARG, std::string("state of '") + names[i] + "' has a different size");
    }
    // 2. states of new names; a failure takes back the ones this call made
    std::vector<std::string> made;
    for (uint32_t i : unknown) {
        auto it = o->states.find(std::string_view(names[i]));
        if (it != o->states.end()) { // the name came up earlier in this call
            if (it->second->numel == numels[i]) continue;
            for (auto &name : made) o->states.erase(name);
            return fail(ERI_ERR_ARG, std::string("state of '") + names[i] + "' has a different size");
        }
        std::unique_ptr<FnState> s(new FnState());
        int rc = s->allocate(numels[i], o->stream, o->state_pool, o->state_lane);
        if (rc) {
            for (auto &name : made) o->states.erase(name);
            return rc;
        }
        made.emplace_back(names[i]);
        o->states.emplace(names[i], std::move(s));
    }
    // 3. rows queued by earlier update() calls keep their place in the order of updates
    int rc = fn_flush(o);
    if (rc) { // their launch failed: nothing of this call has run, and its new states go
        for (auto &name : made) o->states.erase(name);
        return rc;
    }
    for (uint32_t i = 0; i < n; ++i) {
        rc = fn_enqueue(o, names[i], params[i], grads[i], numels[i], dtype_tags[i],
                        grad_dtype_tags ? grad_dtype_tags[i] : dtype_tags[i], outs[i]);
        if (rc) { // only a launch can fail here (a name that repeats flushes the rows before it)
            o->pending.clear();
            o->pending_who.clear();
            o->generation += 1;
            return rc;
        }
    }
    return fn_flush(o);
}

int eri_adam8bit_fn_table_stats(const EriAdam8bitFn *o, uint64_t *flushes, uint64_t *uploads) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (flushes) *flushes = o->flushes;
    if (uploads) *uploads = o->uploads;
    return 0;
}

int eri_adam8bit_fn_set_state_pool(EriAdam8bitFn *o, EriHipPool *pool, uint32_t lane) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    o->state_pool = pool;
    o->state_lane = lane;
    return 0;
}

int eri_adam8bit_fn_set_batching(EriAdam8bitFn *o, int enabled) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    if (!enabled) {
        int rc = fn_flush(o);
        if (rc) return rc;
    }
    o->batching = enabled != 0;
    return 0;
}

int eri_adam8bit_fn_flush(EriAdam8bitFn *o) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    return fn_flush(o);
}

int eri_adam8bit_fn_step(EriAdam8bitFn *o) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    int rc = fn_flush(o); // queued updates belong to the step that ends here (:89-92)
    o->step += 1;
    return rc;
}

int eri_adam8bit_fn_set_lr(EriAdam8bitFn *o, float lr) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    int rc = fn_flush(o); // queued updates were made under the old rate
    o->lr = (double)lr; // `lr as f64`, adam8bit.rs:96
    return rc;
}

uint64_t eri_adam8bit_fn_get_step(const EriAdam8bitFn *o) { return o ? o->step : 0; }

int eri_adam8bit_fn_memory_stats(const EriAdam8bitFn *o, uint64_t *num_params, uint64_t *bytes) {
    if (!o) return fail(ERI_ERR_NULL, "optimizer is NULL");
    uint64_t b = 0;
    for (auto &kv : o->states) b += kv.second->nbytes();
    if (num_params) *num_params = o->states.size();
    if (bytes) *bytes = b;
    return 0;
}

int eri_adam8bit_fn_state_numel(const EriAdam8bitFn *o, const char *name, uint64_t *numel) {
    if (!o || !name || !numel) return fail(ERI_ERR_NULL, "NULL argument");
    auto it = o->states.find(std::string_view(name));
    *numel = it == o->states.end() ? 0 : it->second->numel;
    return 0;
}

int eri_adam8bit_fn_get_state_fp32(EriAdam8bitFn *o, const char *name, float *m_out, float *v_out) {
    if (!o || !name || !m_out || !v_out) return fail(ERI_ERR_NULL, "NULL argument");
    int rc = fn_flush(o);
    if (rc) return rc;
    auto it = o->states.find(std::string_view(name));
    if (it == o->states.end()) return fail(ERI_ERR_ARG, std::string("no optimizer state named '") + name + "'");
    State8 &s = *it->second;
    rc = eri_adam8_dequantize(s.m, s.absmax_m, 1, s.numel, m_out, o->stream);
    if (rc) return rc;
    return eri_adam8_dequantize(s.v, s.absmax_v, 0, s.numel, v_out, o->stream);
}

int eri_adam8bit_fn_load_state_fp32(EriAdam8bitFn *o, const char *name, const float *m, const float *v,
                                    uint64_t numel) {
    if (!o || !name || !m || !v) return fail(ERI_ERR_NULL, "NULL argument");
    if (numel == 0) return fail(ERI_ERR_EMPTY, "InvalidOperation: Empty tensor for quantization");
    int rc = fn_flush(o);
    if (rc) return rc;
    o->last_order.clear(); // it may hold the state that is replaced below
    std::unique_ptr<FnState> s(new FnState());
    rc = s->allocate(numel, o->stream, o->state_pool, o->state_lane);
    if (rc) return rc;
    rc = eri_adam8_quantize(m, 1, numel, s->m, s->absmax_m, o->stream);
    if (rc) return rc;
    rc = eri_adam8_quantize(v, 0, numel, s->v, s->absmax_v, o->stream);
    if (rc) return rc;
    o->states[name] = std::move(s);
    return 0;
}

// ---- helpers beside the optimizers ------------------------------------------------------------

int eri_analyze_optimizer_memory(uint64_t num_params, const char *precision, EriOptimizerMemoryReport *out) {
    if (!precision || !out) return fail(ERI_ERR_NULL, "precision or out is NULL");
    const uint64_t param_bytes = num_params * 4; // adam8bit_enhanced.rs:407
    const std::string p(precision);
    uint64_t state_bytes = param_bytes * 2;
    const char *desc = "Unknown precision";
    if (p == "fp32") { state_bytes = param_bytes * 2; desc = "FP32 momentum states"; }
    else if (p == "fp16") { state_bytes = param_bytes; desc = "FP16 momentum states"; }
    else if (p == "8bit") { state_bytes = param_bytes / 2; desc = "8-bit quantized momentum states"; }
    else if (p == "4bit") { state_bytes = param_bytes / 4; desc = "4-bit quantized momentum states"; }
    const uint64_t total = param_bytes + state_bytes;
    std::memset(out, 0, sizeof(*out));
    out->num_params = num_params;
    out->param_memory_gb = (double)param_bytes / 1e9;
    out->state_memory_gb = (double)state_bytes / 1e9;
    out->total_memory_gb = (double)total / 1e9;
    out->has_reduction = p != "fp32";
    out->memory_reduction_percent =
        out->has_reduction ? (1.0 - (double)total / (double)(param_bytes * 3)) * 100.0 : 0.0; // :419-423
    std::snprintf(out->description, sizeof(out->description), "%s", desc);
    return 0;
}

float eri_ema_decay_from_half_life(uint64_t half_life_steps) { // ema_enhanced.rs:268-272
    return std::pow(0.5f, 1.0f / (float)half_life_steps);
}

float eri_ema_decay_from_window(uint64_t window_size) { // :275-278
    return 1.0f - 2.0f / ((float)window_size + 1.0f);
}

float eri_ema_effective_decay(float decay, uint64_t step, float power, int use_bias_correction) { // :106-127
    float d = decay;
    if (power != 1.0f) {
        const float progress = std::fmin((float)step / 1000.0f, 1.0f);
        d = std::pow(d, power * (1.0f - progress) + progress);
    }
    if (use_bias_correction && step < 1000) {
        const float numerator = 1.0f - std::pow(d, (float)(int32_t)(step - 1));
        const float denominator = 1.0f - std::pow(d, (float)(int32_t)step);
        d = d * numerator / std::fmax(denominator, 1e-8f);
    }
    return d;
}

} // extern "C"

// ---- EMAModel ------------------------------------------------------------------------------------


extern "C" {

int eri_ema_new(float decay, int use_bias_correction, float power, void *stream, EriEmaModel **out) {
    if (!out) return fail(ERI_ERR_NULL, "out is NULL");
    *out = nullptr;
    if (!(0.0f < decay && decay <= 1.0f)) { // ema_enhanced.rs:36-41
        char buf[96];
        std::snprintf(buf, sizeof buf, "InvalidOperation: EMA decay must be in (0, 1], got %g", (double)decay);
        return fail(ERI_ERR_ARG, buf);
    }
    EriEmaModel *e = new EriEmaModel();
    e->decay = decay;
    e->bias_correction = use_bias_correction != 0;
    e->power = power;
    e->stream = stream;
    *out = e;
    return 0;
}

int eri_ema_destroy(EriEmaModel *e) {
    delete e;
    return 0;
}

int eri_ema_init_from_params(EriEmaModel *e, const char *const *names, EriParameter *const *params, uint32_t n) {
    if (!e || (n && (!names || !params))) return fail(ERI_ERR_NULL, "NULL argument");
    for (uint32_t i = 0; i < n; ++i) {
        if (!names[i]) return fail(ERI_ERR_NULL, "NULL name");
        int rc = ema_adopt(e, names[i], params[i]);
        if (rc) return rc;
    }
    return 0;
}

uint64_t eri_ema_step(const EriEmaModel *e) { return e ? e->step : 0; }

int eri_ema_set_step(EriEmaModel *e, uint64_t step) {
    if (!e) return fail(ERI_ERR_NULL, "ema is NULL");
    e->step = step;
    return 0;
}

float eri_ema_current_decay(const EriEmaModel *e) {
    return e ? eri_ema_effective_decay(e->decay, e->step, e->power, e->bias_correction) : 0.0f;
}

uint32_t eri_ema_num_shadows(const EriEmaModel *e) { return e ? (uint32_t)e->shadows.size() : 0; }

int eri_ema_shadow(const EriEmaModel *e, const char *name, void **data, uint64_t *numel, int *dtype_tag) {
    if (!e || !name) return fail(ERI_ERR_NULL, "NULL argument");
    auto it = e->shadows.find(name);
    if (it == e->shadows.end()) return fail(ERI_ERR_ARG, std::string("InvalidOperation: No EMA weights found for parameter: ") + name);
    if (data) *data = it->second.data;
    if (numel) *numel = it->second.numel;
    if (dtype_tag) *dtype_tag = it->second.dtype;
    return 0;
}

int eri_ema_update(EriEmaModel *e, const char *const *names, EriParameter *const *params, uint32_t n) {
    if (!e || (n && (!names || !params))) return fail(ERI_ERR_NULL, "NULL argument");
    for (uint32_t i = 0; i < n; ++i)
        if (!names[i] || !params[i] || !params[i]->data) return fail(ERI_ERR_NULL, "NULL name or parameter");
    e->step += 1;                                      // ema_enhanced.rs:80
    const float d = eri_ema_current_decay(e);           // :83
    e->rows.clear();
    for (uint32_t i = 0; i < n; ++i) {
        auto it = e->shadows.find(names[i]);
        const EriParameter *p = params[i];
        if (it == e->shadows.end() || it->second.numel != p->numel || it->second.dtype != p->dtype) {
            int rc = ema_adopt(e, names[i], p);          // :100-103 first time seeing this parameter
            if (rc) return rc;
            continue;
        }
        EriEmaTensor r;
        r.shadow = it->second.data;
        r.p = p->data;
        r.numel = p->numel;
        r.dtype_tag = p->dtype;
        r.reserved = 0;
        e->rows.push_back(r);
    }
    if (e->rows.empty()) return 0;
    return eri_ema_update_multi(e->rows.data(), (uint32_t)e->rows.size(), d, e->stream); // :88-98
}

int eri_ema_copy_to(EriEmaModel *e, const char *const *names, EriParameter *const *params, uint32_t n) {
    if (!e || (n && (!names || !params))) return fail(ERI_ERR_NULL, "NULL argument");
    for (uint32_t i = 0; i < n; ++i) { // refuse before anything is copied
        if (!names[i] || !params[i] || !params[i]->data) return fail(ERI_ERR_NULL, "NULL name or parameter");
        auto it = e->shadows.find(names[i]);
        if (it == e->shadows.end())
            return fail(ERI_ERR_ARG, std::string("InvalidOperation: No EMA weights found for parameter: ") + names[i]);
        if (it->second.numel != params[i]->numel || it->second.dtype != params[i]->dtype)
            return fail(ERI_ERR_ARG, std::string("EMA weights do not fit parameter: ") + names[i]);
    }
    for (uint32_t i = 0; i < n; ++i) {
        const EriEmaModel::Shadow &s = e->shadows[names[i]];
        int rc = eri_hip_memcpy_async(params[i]->data, s.data, s.numel * elem_bytes(s.dtype), 3, e->stream);
        if (rc) return rc;
    }
    return 0;
}

} // extern "C"
