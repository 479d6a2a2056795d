/*
 * A parity check written against the C ABI alone: no Python, no torch.  It allocates through
 * eri_hip_*, runs optimizer steps on the device through include/eri_optim8.h and the same steps through
 * the CPU oracle (oracle/adam8_oracle.c, linked as liberi_oracle.so), and compares parameters, codes and
 * absmax bit for bit.  This is what a maintainer binding the library from C, Rust or Go sees.
 * Test infrastructure: built by tests/Makefile, run by tests/test_gpu_cabi_c.py on a machine with a GPU.
 *
 * usage: cabi_parity [bf16|f32] [eri|l2|bnb]
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

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

static uint32_t rng_state = 0x9E3779B9u;
static float rnd_normal(void) { /* sum of twelve uniforms minus six */
    float s = 0.0f;
    for (int i = 0; i < 12; ++i) {
        rng_state = rng_state * 1664525u + 1013904223u;
        s += (float)(rng_state >> 8) * (1.0f / 16777216.0f);
    }
    return s - 6.0f;
}

enum { N_TENSORS = 5, STEPS = 3 };

int main(int argc, char **argv) {
    const int bf16 = !(argc > 1 && strcmp(argv[1], "f32") == 0);
    int mode = ERI_ADAM8_MODE_ERI;
    if (argc > 2 && strcmp(argv[2], "l2") == 0) mode = ERI_ADAM8_MODE_L2;
    if (argc > 2 && strcmp(argv[2], "bnb") == 0) mode = ERI_ADAM8_MODE_BNB;
    const uint64_t sizes[N_TENSORS] = {2048 * 5 + 40, 320, 2048, 7, 40000};
    const size_t esz = bf16 ? 2 : 4;
    const int tag = bf16 ? ERI_DTYPE_BF16 : ERI_DTYPE_F32;
    float map_s[256], map_u[256];
    CHECK(eri_adam8_get_maps(map_s, map_u));

    void *stream = NULL;
    CHECK(eri_hip_stream_create(&stream));
    EriAdam8Tensor rows[N_TENSORS];
    void *hp[N_TENSORS], *hg[N_TENSORS];
    uint8_t *hm[N_TENSORS], *hv[N_TENSORS];
    float *ham[N_TENSORS], *hav[N_TENSORS];
    uint64_t start = 0;
    for (int i = 0; i < N_TENSORS; ++i) {
        const uint64_t n = sizes[i], nb = (n + 2047) / 2048;
        hp[i] = malloc(n * esz); hg[i] = malloc(n * esz);
        hm[i] = malloc(n); hv[i] = malloc(n);
        ham[i] = malloc(nb * 4); hav[i] = malloc(nb * 4);
        for (uint64_t k = 0; k < n; ++k) {
            const float x = rnd_normal() * 0.02f;
            if (bf16) ((uint16_t *)hp[i])[k] = eri_oracle_f32_to_bf16(x); else ((float *)hp[i])[k] = x;
        }
        eri_oracle_state_init(hm[i], hv[i], ham[i], hav[i], n);
        EriAdam8Tensor *r = &rows[i];
        memset(r, 0, sizeof *r);
        CHECK(eri_hip_malloc_zeroed(0, n * esz, &r->p));
        CHECK(eri_hip_malloc_zeroed(0, n * esz, (void **)&r->g));
        CHECK(eri_hip_malloc_zeroed(0, n, (void **)&r->m));
        CHECK(eri_hip_malloc_zeroed(0, n, (void **)&r->v));
        CHECK(eri_hip_malloc_zeroed(0, nb * 4, (void **)&r->absmax_m));
        CHECK(eri_hip_malloc_zeroed(0, nb * 4, (void **)&r->absmax_v));
        r->numel = n; r->block_start = start; r->dtype_tag = tag; r->grad_scale = 1.0f;
        start += nb;
        CHECK(eri_hip_memcpy_async(r->p, hp[i], n * esz, 1, stream));
        CHECK(eri_adam8_state_init(r->m, r->v, r->absmax_m, r->absmax_v, n, stream));
    }
    EriAdam8Table *table = NULL;
    CHECK(eri_adam8_table_create(rows, N_TENSORS, stream, &table));
    for (int t = 0; t < STEPS; ++t) {
        const uint64_t step = mode == ERI_ADAM8_MODE_L2 ? (uint64_t)t : (uint64_t)t + 1;
        EriAdam8Hyper h;
        CHECK(eri_adam8_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, step, mode, ERI_ADAM8_FLAG_EXACT_PARAM, &h));
        EriOracleHyper ho;
        eri_oracle_hyper_pack(1e-4, 0.9, 0.999, 1e-8, 0.01, step, mode, &ho);
        for (int i = 0; i < N_TENSORS; ++i) {
            const uint64_t n = sizes[i];
            for (uint64_t k = 0; k < n; ++k) {
                const float x = rnd_normal() * 1e-3f;
                if (bf16) ((uint16_t *)hg[i])[k] = eri_oracle_f32_to_bf16(x); else ((float *)hg[i])[k] = x;
            }
            CHECK(eri_hip_memcpy_async((void *)rows[i].g, hg[i], n * esz, 1, stream));
            if (eri_oracle_step_tensor(hp[i], hg[i], hm[i], hv[i], ham[i], hav[i], n, tag, &ho, map_s, map_u, 1) != 0) return 3;
        }
        CHECK(eri_hip_stream_sync(stream)); /* the host gradient buffers are reused next step */
        CHECK(eri_adam8_step_table(table, &h, stream));
    }
    int bad = 0;
    for (int i = 0; i < N_TENSORS; ++i) {
        const uint64_t n = sizes[i], nb = (n + 2047) / 2048;
        void *gp = malloc(n * esz); uint8_t *gm = malloc(n), *gv = malloc(n);
        float *gam = malloc(nb * 4), *gav = malloc(nb * 4);
        CHECK(eri_hip_memcpy_async(gp, rows[i].p, n * esz, 2, stream));
        CHECK(eri_hip_memcpy_async(gm, rows[i].m, n, 2, stream));
        CHECK(eri_hip_memcpy_async(gv, rows[i].v, n, 2, stream));
        CHECK(eri_hip_memcpy_async(gam, rows[i].absmax_m, nb * 4, 2, stream));
        CHECK(eri_hip_memcpy_async(gav, rows[i].absmax_v, nb * 4, 2, stream));
        CHECK(eri_hip_stream_sync(stream));
        const int same = memcmp(gp, hp[i], n * esz) == 0 && memcmp(gm, hm[i], n) == 0 && memcmp(gv, hv[i], n) == 0 &&
                         memcmp(gam, ham[i], nb * 4) == 0 && memcmp(gav, hav[i], nb * 4) == 0;
        printf("tensor %d (%llu elements): %s\n", i, (unsigned long long)n, same ? "bit-exact" : "DIFFERS");
        bad += !same;
        free(gp); free(gm); free(gv); free(gam); free(gav);
    }
    CHECK(eri_adam8_table_destroy(table));
    for (int i = 0; i < N_TENSORS; ++i) {
        eri_hip_free(rows[i].p); eri_hip_free((void *)rows[i].g); eri_hip_free(rows[i].m); eri_hip_free(rows[i].v);
        eri_hip_free(rows[i].absmax_m); eri_hip_free(rows[i].absmax_v);
        free(hp[i]); free(hg[i]); free(hm[i]); free(hv[i]); free(ham[i]); free(hav[i]);
    }
    CHECK(eri_hip_stream_destroy(stream));
    printf("%s %s: %s\n", bf16 ? "bf16" : "f32", mode == 0 ? "eri" : mode == 1 ? "l2" : "bnb", bad ? "FAILED" : "ok");
    return bad ? 1 : 0;
}
