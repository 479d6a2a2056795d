/*
 * A trainer's optimizer calls written in plain C against include/eri_adam8bit.h alone: the list optimizer
 * (Adam8bit::new / step, adam8bit_enhanced.rs:161-291) and the functional optimizer (Adam8bit::with_params /
 * update / step, adam8bit.rs:69-208), with parameters, gradients and optimizer state taken from three lanes of
 * the library's device pool.  Every step also runs through the CPU oracle (oracle/adam8_oracle.c, linked as
 * liberi_oracle.so), and parameters, codes and absmax are compared bit for bit.  No Python, no torch: this is
 * the view of a maintainer who binds the objects from C, Rust or Go.
 * Test infrastructure: built by tests/Makefile, run by tests/test_gpu_cabi_c.py on a machine with a GPU.
 *
 * usage: cabi_objects [bf16|f32] [list|functional]
 */
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "eri_adam8bit.h"
#include "eri_optim8.h"

/* the oracle's interface (oracle/adam8_oracle.c) */
typedef struct EriOracleHyper {
    float beta1, beta2, omb1, omb2, eps, weight_decay, step_size, bc1, bc2, grad_scale;
    int32_t mode, use_grad_scale;
} EriOracleHyper;
void eri_oracle_hyper_pack(double lr, double beta1, double beta2, double eps, double wd, uint64_t step, int mode, EriOracleHyper *h);
int eri_oracle_step_tensor(void *p, const void *g, uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel,
                           int dtype, const EriOracleHyper *h, const float *map_s, const float *map_u, int threads);
void eri_oracle_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel);
uint16_t eri_oracle_f32_to_bf16(float f);

#define CHECK(call)                                                                        \
    do {                                                                                   \
        int rc_ = (call);                                                                  \
        if (rc_ != 0) {                                                                    \
            fprintf(stderr, "%s failed with code %d: %s\n", #call, rc_, eri_last_error()); \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)

static uint32_t rng_state = 0x51F15EEDu;
static float rnd_normal(void) { /* sum of twelve uniforms minus six */
    float s = 0.0f;
    for (int i = 0; i < 12; ++i) {
        rng_state = rng_state * 1664525u + 1013904223u;
        s += (float)(rng_state >> 8) * (1.0f / 16777216.0f);
    }
    return s - 6.0f;
}

enum { N_TENSORS = 4, STEPS = 3 };
static const uint64_t kSizes[N_TENSORS] = {2048 * 3 + 100, 2048 * 8, 999, 2048 * 2 + 2047};
static const char *const kNames[N_TENSORS] = {"lora_a.0", "lora_b.0", "lora_a.1", "lora_b.1"};

typedef struct Host { /* the oracle's side of one tensor */
    void *p, *g;
    uint8_t *m, *v;
    float *am, *av;
} Host;

static void fill(void *dst, uint64_t n, float std, int bf16) {
    for (uint64_t k = 0; k < n; ++k) {
        const float x = rnd_normal() * std;
        if (bf16) ((uint16_t *)dst)[k] = eri_oracle_f32_to_bf16(x);
        else ((float *)dst)[k] = x;
    }
}

/* parameters and 8-bit state on the device against the oracle's */
static int same_as_oracle(const Host *h, uint64_t n, size_t esz, const void *dp, const uint8_t *dm, const uint8_t *dv,
                          const float *dam, const float *dav, void *stream) {
    const uint64_t nb = (n + 2047) / 2048;
    void *gp = malloc(n * esz);
    uint8_t *gm = malloc(n), *gv = malloc(n);
    float *gam = malloc(nb * 4), *gav = malloc(nb * 4);
    int ok = eri_hip_memcpy_async(gp, dp, n * esz, 2, stream) == 0 && eri_hip_memcpy_async(gm, dm, n, 2, stream) == 0 &&
             eri_hip_memcpy_async(gv, dv, n, 2, stream) == 0 && eri_hip_memcpy_async(gam, dam, nb * 4, 2, stream) == 0 &&
             eri_hip_memcpy_async(gav, dav, nb * 4, 2, stream) == 0 && eri_hip_stream_sync(stream) == 0;
    ok = ok && memcmp(gp, h->p, n * esz) == 0 && memcmp(gm, h->m, n) == 0 && memcmp(gv, h->v, n) == 0 &&
         memcmp(gam, h->am, nb * 4) == 0 && memcmp(gav, h->av, nb * 4) == 0;
    free(gp); free(gm); free(gv); free(gam); free(gav);
    return ok;
}

int main(int argc, char **argv) {
    const int bf16 = !(argc > 1 && strcmp(argv[1], "f32") == 0);
    const int functional = argc > 2 && strcmp(argv[2], "functional") == 0;
    const size_t esz = bf16 ? 2 : 4;
    const int tag = bf16 ? ERI_DTYPE_BF16 : ERI_DTYPE_F32;
    const double lr = 1e-4, b1 = 0.9, b2 = 0.999, eps = 1e-8, wd = 0.01;
    float map_s[256], map_u[256];
    CHECK(eri_adam8_get_maps(map_s, map_u));

    void *stream = NULL;
    CHECK(eri_hip_stream_create(&stream));
    /* four lanes of 64 MiB: parameters in lane 0, gradients in lane 1, optimizer state in lane 2 */
    EriHipPool *pool = NULL;
    CHECK(eri_hip_pool_create(0, (size_t)256 << 20, 4, &pool));

    Host host[N_TENSORS];
    void *dp[N_TENSORS], *dp2[N_TENSORS], *dg[N_TENSORS];
    for (int i = 0; i < N_TENSORS; ++i) {
        const uint64_t n = kSizes[i], nb = (n + 2047) / 2048;
        host[i].p = malloc(n * esz); host[i].g = malloc(n * esz);
        host[i].m = malloc(n); host[i].v = malloc(n);
        host[i].am = malloc(nb * 4); host[i].av = malloc(nb * 4);
        fill(host[i].p, n, 0.02f, bf16);
        eri_oracle_state_init(host[i].m, host[i].v, host[i].am, host[i].av, n);
        CHECK(eri_hip_pool_alloc_zeroed(pool, 0, n * esz, &dp[i]));
        CHECK(eri_hip_pool_alloc_zeroed(pool, 0, n * esz, &dp2[i])); /* the functional update's other output set */
        CHECK(eri_hip_pool_alloc_zeroed(pool, 1, n * esz, &dg[i]));
        CHECK(eri_hip_memcpy_async(dp[i], host[i].p, n * esz, 1, stream));
    }
    CHECK(eri_hip_stream_sync(stream));
    int bad = 0;

    if (!functional) {
        EriParameter *params[N_TENSORS];
        for (int i = 0; i < N_TENSORS; ++i) CHECK(eri_param_create(dp[i], kSizes[i], tag, &params[i]));
        EriAdam8bitConfig cfg;
        eri_adam8bit_config_default(&cfg);
        cfg.lr = lr; cfg.beta1 = b1; cfg.beta2 = b2; cfg.eps = eps; cfg.weight_decay = wd;
        EriAdam8bit *opt = NULL;
        CHECK(eri_adam8bit_new(params, N_TENSORS, &cfg, stream, &opt));
        CHECK(eri_adam8bit_set_state_pool(opt, pool, 2));
        /* no eri_adam8bit_set_flags: a new optimizer reproduces the reference's bf16 parameters bit for bit */
        for (int t = 1; t <= STEPS; ++t) {
            EriOracleHyper ho;
            eri_oracle_hyper_pack(lr, b1, b2, eps, wd, (uint64_t)t, ERI_ADAM8_MODE_ERI, &ho);
            uint32_t want_skipped = 0;
            for (int i = 0; i < N_TENSORS; ++i) {
                const int has_grad = !(t == 2 && i == 2); /* one parameter sits out the second step */
                if (!has_grad) {
                    CHECK(eri_param_set_grad(params[i], NULL));
                    ++want_skipped;
                    continue;
                }
                fill(host[i].g, kSizes[i], 1e-3f, bf16);
                CHECK(eri_hip_memcpy_async(dg[i], host[i].g, kSizes[i] * esz, 1, stream));
                CHECK(eri_param_set_grad(params[i], dg[i]));
                if (eri_oracle_step_tensor(host[i].p, host[i].g, host[i].m, host[i].v, host[i].am, host[i].av, kSizes[i], tag,
                                           &ho, map_s, map_u, 1) != 0) return 3;
            }
            CHECK(eri_hip_stream_sync(stream)); /* the host gradient buffers are refilled next step */
            uint32_t skipped = 99;
            CHECK(eri_adam8bit_step(opt, &skipped));
            if (skipped != want_skipped) { printf("step %d skipped %u parameters, expected %u\n", t, skipped, want_skipped); ++bad; }
        }
        if (eri_adam8bit_get_step(opt) != STEPS) { printf("step counter reads %llu\n", (unsigned long long)eri_adam8bit_get_step(opt)); ++bad; }
        uint64_t want_bytes = 0;
        for (int i = 0; i < N_TENSORS; ++i) {
            uint8_t *m, *v;
            float *am, *av;
            CHECK(eri_adam8bit_state_ptrs(opt, (uint32_t)i, &m, &v, &am, &av));
            const int same = m && same_as_oracle(&host[i], kSizes[i], esz, dp[i], m, v, am, av, stream);
            printf("parameter %d (%llu elements): %s\n", i, (unsigned long long)kSizes[i], same ? "bit-exact" : "DIFFERS");
            bad += !same;
            want_bytes += 2 * kSizes[i] + 8 * ((kSizes[i] + 2047) / 2048);
        }
        if (eri_adam8bit_quantized_memory_usage(opt) != want_bytes) { printf("quantized_memory_usage differs\n"); ++bad; }
        size_t used = 0;
        CHECK(eri_hip_pool_lane_used(pool, 2, &used));
        if (used < want_bytes) { printf("the states did not come out of lane 2 (%zu bytes used there)\n", used); ++bad; }
        CHECK(eri_adam8bit_destroy(opt));
        for (int i = 0; i < N_TENSORS; ++i) CHECK(eri_param_release(params[i]));
    } else {
        EriAdam8bitFn *opt = NULL;
        CHECK(eri_adam8bit_fn_with_params(lr, b1, b2, eps, wd, stream, &opt));
        CHECK(eri_adam8bit_fn_set_state_pool(opt, pool, 2));
        const void *in[N_TENSORS], *grads[N_TENSORS];
        void *out[N_TENSORS];
        int32_t tags[N_TENSORS];
        for (int i = 0; i < N_TENSORS; ++i) tags[i] = tag;
        for (int t = 0; t < STEPS; ++t) {
            /* update() returns a new tensor: the output of one step is the input of the next */
            for (int i = 0; i < N_TENSORS; ++i) {
                in[i] = (t & 1) ? dp2[i] : dp[i];
                out[i] = (t & 1) ? dp[i] : dp2[i];
                grads[i] = dg[i];
            }
            EriOracleHyper ho; /* the counter is bumped after the updates (adam8bit.rs:89-92, :164) */
            eri_oracle_hyper_pack(lr, b1, b2, eps, wd, eri_adam8bit_fn_get_step(opt), ERI_ADAM8_MODE_L2, &ho);
            for (int i = 0; i < N_TENSORS; ++i) {
                fill(host[i].g, kSizes[i], 1e-3f, bf16);
                CHECK(eri_hip_memcpy_async(dg[i], host[i].g, kSizes[i] * esz, 1, stream));
                if (eri_oracle_step_tensor(host[i].p, host[i].g, host[i].m, host[i].v, host[i].am, host[i].av, kSizes[i], tag,
                                           &ho, map_s, map_u, 1) != 0) return 3;
            }
            CHECK(eri_hip_stream_sync(stream));
            CHECK(eri_adam8bit_fn_update_many(opt, kNames, in, grads, kSizes, tags, NULL, out, N_TENSORS));
            CHECK(eri_adam8bit_fn_step(opt));
        }
        if (eri_adam8bit_fn_get_step(opt) != STEPS) { printf("step counter reads %llu\n", (unsigned long long)eri_adam8bit_fn_get_step(opt)); ++bad; }
        uint64_t flushes = 0, uploads = 0;
        CHECK(eri_adam8bit_fn_table_stats(opt, &flushes, &uploads));
        /* three launches over two alternating sets of rows: the third finds its table */
        if (flushes != STEPS || uploads != 2) { printf("%llu launches, %llu table uploads\n", (unsigned long long)flushes, (unsigned long long)uploads); ++bad; }
        for (int i = 0; i < N_TENSORS; ++i) {
            /* the moments as fp32 (get_state_as_tensors, adam8bit.rs:296-308: device tensors) against the
             * oracle's codes */
            const uint64_t n = kSizes[i];
            float *m32 = malloc(n * 4), *v32 = malloc(n * 4);
            void *dm32 = NULL, *dv32 = NULL;
            CHECK(eri_hip_pool_alloc_zeroed(pool, 3, n * 4, &dm32));
            CHECK(eri_hip_pool_alloc_zeroed(pool, 3, n * 4, &dv32));
            /* ordinary host memory must be refused before any kernel sees it; the call is only made once the
             * runtime has said that it tells the two kinds of buffer apart */
            int kind_host = -1, kind_dev = -1;
            CHECK(eri_hip_pointer_kind(m32, &kind_host));
            CHECK(eri_hip_pointer_kind(dm32, &kind_dev));
            if (kind_host != ERI_PTR_UNKNOWN || kind_dev != ERI_PTR_DEVICE) {
                printf("pointer kinds: host buffer %d, device buffer %d\n", kind_host, kind_dev);
                return 4;
            }
            if (eri_adam8bit_fn_get_state_fp32(opt, kNames[i], m32, v32) != ERI_ERR_ARG) {
                printf("get_state_fp32 did not refuse host buffers\n");
                return 4;
            }
            CHECK(eri_adam8bit_fn_get_state_fp32(opt, kNames[i], (float *)dm32, (float *)dv32));
            CHECK(eri_hip_memcpy_async(m32, dm32, n * 4, 2, stream));
            CHECK(eri_hip_memcpy_async(v32, dv32, n * 4, 2, stream));
            CHECK(eri_hip_stream_sync(stream));
            int same = 1;
            for (uint64_t k = 0; k < n && same; ++k) {
                const float wm = map_s[host[i].m[k]] * host[i].am[k / 2048], wv = map_u[host[i].v[k]] * host[i].av[k / 2048];
                same = memcmp(&wm, &m32[k], 4) == 0 && memcmp(&wv, &v32[k], 4) == 0;
            }
            void *gp = malloc(n * esz);
            CHECK(eri_hip_memcpy_async(gp, (STEPS & 1) ? dp2[i] : dp[i], n * esz, 2, stream));
            CHECK(eri_hip_stream_sync(stream));
            same = same && memcmp(gp, host[i].p, n * esz) == 0;
            printf("parameter %d (%llu elements): %s\n", i, (unsigned long long)n, same ? "bit-exact" : "DIFFERS");
            bad += !same;
            free(gp); free(m32); free(v32);
        }
        CHECK(eri_adam8bit_fn_destroy(opt));
    }

    CHECK(eri_hip_pool_destroy(pool));
    CHECK(eri_hip_stream_destroy(stream));
    for (int i = 0; i < N_TENSORS; ++i) {
        free(host[i].p); free(host[i].g); free(host[i].m); free(host[i].v); free(host[i].am); free(host[i].av);
    }
    printf("%s %s: %s\n", bf16 ? "bf16" : "f32", functional ? "functional" : "list", bad ? "FAILED" : "ok");
    return bad ? 1 : 0;
}
