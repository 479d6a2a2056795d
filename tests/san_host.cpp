/*
 * The host side of the library under AddressSanitizer and UndefinedBehaviorSanitizer, without a GPU: the two
 * host translation units (the C ABI and the optimizer objects) are rebuilt with the sanitizers into
 * tests/_san/libsan_host.so, which stands in front of the product library (the kernels' launchers come from
 * there and are never reached), and this program drives the code that handles untrusted bytes and caller
 * mistakes: the state-file parsers over a directory of mutated files, row validation, the functional
 * optimizer's queue, the pool's book-keeping arguments.  Every call must come back with a return code.
 * Test infrastructure: built by tests/san_host.mk, run by tests/test_host_sanitizers.py.
 *
 * usage: san_host <directory with NNN.st (safetensors) and NNN.bc (bincode) files> <count>
 */
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "eri_adam8bit.h"
#include "eri_optim8.h"

static int failures = 0;
#define EXPECT(cond)                                                        \
    do {                                                                    \
        if (!(cond)) {                                                      \
            std::printf("line %d: %s does not hold (%s)\n", __LINE__, #cond, eri_last_error()); \
            ++failures;                                                     \
        }                                                                   \
    } while (0)

static void *fake(uintptr_t a) { return reinterpret_cast<void *>(a); } // addresses that are never dereferenced

int main(int argc, char **argv) {
    if (argc < 3) return 2;
    const std::string dir = argv[1];
    const int count = std::atoi(argv[2]);

    // ---- state files: every mutation comes back with a code, and a refused file leaves the optimizer as it was
    EriParameter *ps[2] = {nullptr, nullptr};
    for (int i = 0; i < 2; ++i) EXPECT(eri_param_create(fake(0x10000 * (i + 1)), 4096, ERI_DTYPE_BF16, &ps[i]) == 0);
    EriAdam8bit *opt = nullptr;
    EXPECT(eri_adam8bit_new(ps, 2, nullptr, nullptr, &opt) == 0);
    int refused = 0;
    for (int k = 0; k < count; ++k) {
        char name[32];
        std::snprintf(name, sizeof name, "/%03d.%s", k, k % 2 == 0 ? "st" : "bc");
        const std::string path = dir + name;
        const int rc = k % 2 == 0 ? eri_adam8bit_load_state(opt, path.c_str()) : eri_adam8bit_load_legacy_state(opt, path.c_str());
        if (rc == ERI_ERR_ARG) {
            ++refused;
            EXPECT(eri_adam8bit_get_step(opt) == 0);
        }
        EXPECT(rc != 0 || true); // a file that parses goes on to the device upload, which has no device here
    }
    std::printf("%d of %d files refused by the parsers\n", refused, count);
    EXPECT(refused > count / 2);
    EXPECT(eri_adam8bit_load_state(opt, (dir + "/missing").c_str()) == ERI_ERR_ARG);
    EXPECT(eri_adam8bit_save_state(opt, (dir + "/no/such/dir/state").c_str()) != 0);
    uint32_t skipped = 0;
    EXPECT(eri_adam8bit_step(opt, &skipped) == 0 && skipped == 2); // no gradients: nothing to launch
    EXPECT(eri_adam8bit_set_param_grad_scale(opt, 7, 1.0f) == ERI_ERR_ARG);
    EXPECT(eri_adam8bit_set_mode(opt, 9) == ERI_ERR_ARG);
    EXPECT(eri_adam8bit_destroy(opt) == 0);
    for (auto *p : ps) EXPECT(eri_param_release(p) == 0);

    // ---- launch-table rows: each mistake is named before anything touches a device
    std::vector<EriAdam8Tensor> rows(3);
    std::memset(rows.data(), 0, rows.size() * sizeof(EriAdam8Tensor));
    uint64_t start = 0;
    for (size_t i = 0; i < rows.size(); ++i) {
        EriAdam8Tensor &r = rows[i];
        r.p = fake(0x100000 * (i + 1));
        r.g = fake(0x200000 * (i + 1));
        r.m = static_cast<uint8_t *>(fake(0x300000 * (i + 1)));
        r.v = static_cast<uint8_t *>(fake(0x400000 * (i + 1)));
        r.absmax_m = static_cast<float *>(fake(0x500000 * (i + 1)));
        r.absmax_v = static_cast<float *>(fake(0x600000 * (i + 1)));
        r.numel = 5000 + 100 * i;
        r.block_start = start;
        r.dtype_tag = ERI_DTYPE_BF16;
        r.grad_scale = 1.0f;
        start += (r.numel + 2047) / 2048;
    }
    EriAdam8Table *table = nullptr;
    EXPECT(eri_adam8_table_create(nullptr, 3, nullptr, &table) == ERI_ERR_NULL);
    EXPECT(eri_adam8_table_create(rows.data(), 0, nullptr, &table) == ERI_ERR_ARG);
    {
        auto bad = rows;
        bad[1].p = fake(0x100008);
        EXPECT(eri_adam8_table_create(bad.data(), 3, nullptr, &table) == ERI_ERR_ALIGN);
        bad = rows;
        bad[2].numel = 0;
        EXPECT(eri_adam8_table_create(bad.data(), 3, nullptr, &table) == ERI_ERR_EMPTY);
        bad = rows;
        bad[0].dtype_tag = 7;
        EXPECT(eri_adam8_table_create(bad.data(), 3, nullptr, &table) == ERI_ERR_DTYPE);
        bad = rows;
        bad[2].block_start += 1;
        EXPECT(eri_adam8_table_create(bad.data(), 3, nullptr, &table) == ERI_ERR_BLOCK_START);
        bad = rows;
        bad[1].v = nullptr;
        EXPECT(eri_adam8_table_create(bad.data(), 3, nullptr, &table) == ERI_ERR_NULL);
    }
    EriAdam8Hyper h;
    EXPECT(eri_adam8_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, 3, ERI_ADAM8_MODE_ERI, 0, &h) == 0);
    EXPECT(eri_adam8_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, 3, 5, 0, &h) == ERI_ERR_ARG);
    EXPECT(eri_adam8_step_table(nullptr, &h, nullptr) == ERI_ERR_NULL);
    float maps[2][256];
    EXPECT(eri_adam8_get_maps(maps[0], maps[1]) == 0 && maps[0][127] == 0.0f && maps[1][255] == 1.0f);
    std::vector<char> image(1 << 18);
    size_t bytes = 0;
    uint32_t offsets[6];
    EXPECT(eri_adam8_table_image(image.data(), image.size(), &bytes, offsets) == 0 && bytes > 4096 && bytes <= image.size());
    EXPECT(eri_adam8_table_image(image.data(), 100, &bytes, offsets) != 0);

    // ---- the functional optimizer's queue: refused rows leave nothing behind
    EriAdam8bitFn *fn = nullptr;
    EXPECT(eri_adam8bit_fn_with_params(1e-4, 0.9, 0.999, 1e-8, 0.01, nullptr, &fn) == 0);
    EXPECT(eri_adam8bit_fn_update(fn, nullptr, fake(0x1000), fake(0x2000), 64, ERI_DTYPE_BF16, ERI_DTYPE_BF16, fake(0x3000)) == ERI_ERR_NULL);
    EXPECT(eri_adam8bit_fn_update(fn, "w", fake(0x1000), fake(0x2000), 0, ERI_DTYPE_BF16, ERI_DTYPE_BF16, fake(0x3000)) == ERI_ERR_EMPTY);
    EXPECT(eri_adam8bit_fn_update(fn, "w", fake(0x1004), fake(0x2000), 64, ERI_DTYPE_BF16, ERI_DTYPE_BF16, fake(0x3000)) == ERI_ERR_ALIGN);
    const char *names[2] = {"a", "b"};
    const void *in[2] = {fake(0x1000), fake(0x1008)}, *gr[2] = {fake(0x2000), fake(0x4000)};
    void *out[2] = {fake(0x5000), fake(0x6000)};
    const uint64_t numels[2] = {64, 64};
    const int32_t tags[2] = {ERI_DTYPE_BF16, ERI_DTYPE_BF16};
    EXPECT(eri_adam8bit_fn_update_many(fn, names, in, gr, numels, tags, nullptr, out, 2) == ERI_ERR_ALIGN);
    uint64_t n_states = 99, state_bytes = 99;
    EXPECT(eri_adam8bit_fn_memory_stats(fn, &n_states, &state_bytes) == 0 && n_states == 0 && state_bytes == 0);
    uint64_t numel = 99;
    EXPECT(eri_adam8bit_fn_state_numel(fn, "a", &numel) == 0 && numel == 0);
    EXPECT(eri_adam8bit_fn_step(fn) == 0 && eri_adam8bit_fn_get_step(fn) == 1);
    EXPECT(eri_adam8bit_fn_destroy(fn) == 0);

    // ---- helpers with no device behind them
    EriOptimizerMemoryReport rep;
    EXPECT(eri_analyze_optimizer_memory(1000000, "8bit", &rep) == 0);
    EXPECT(eri_analyze_optimizer_memory(1000000, nullptr, &rep) == ERI_ERR_NULL);
    EXPECT(eri_ema_effective_decay(0.999f, 10, 1.0f, 1) > 0.0f);
    EXPECT(eri_hip_pool_release(nullptr, fake(0x1000), 256) == ERI_ERR_NULL);
    EXPECT(eri_hip_pool_destroy(nullptr) == 0);

    std::printf("%s\n", failures ? "FAILED" : "ok");
    return failures ? 1 : 0;
}
