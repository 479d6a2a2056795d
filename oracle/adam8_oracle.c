/*
 * CPU oracle for the blockwise 8-bit AdamW step.  TEST INFRASTRUCTURE ONLY: nothing in the
 * shipped library or the Python package may link, load or call this file; it exists so that the
 * tests, the smoke check and the benchmark's cpu_baseline leg have something to compare with
 * and to time.
 *
 * It is a scalar restatement, one individually rounded fp32 operation per line, of
 *   - EriDiffusion's Adam8bit::step          src/trainers/adam8bit_enhanced.rs:202-291  (mode ERI)
 *   - EriDiffusion's functional Adam8bit::update  src/trainers/adam8bit.rs:101-208      (mode L2)
 *   - mode BNB: the parameter update and the sign rule of the library the state format comes from
 *     (bitsandbytes 8-bit blockwise Adam, csrc/kernels.cu kOptimizerStatic8bit2StateBlockwise; not
 *     installed here, not used by the reference): eps scaled by sqrt(bc2), decay applied as a
 *     factor (1 - lr*wd) after the Adam term, and a first-moment code whose map value has the
 *     other sign than the moment moved one entry toward the moment's sign
 * with the state held in the blockwise format the optimizer is specified to use: uint8 codes
 * into the signed (first moment) and unsigned (second moment) 256-entry dynamic maps of
 * bitsandbytes (functional.py: create_dynamic_map), one fp32 absmax per 2048-element block.
 * The reference tree has no blockwise quantiser and no golden vectors for any optimizer, so the
 * quantiser half of this file restates the published bitsandbytes blockwise algorithm
 * (quantize_blockwise / dequantize_blockwise: code -> map[code] * absmax, value -> nearest map
 * entry of value / absmax); what pins it is listed next to each function.
 *
 * Pinning status (tests/test_oracle_*.py):
 *   eri_oracle_bf16_*          all 65,536 high halves against torch.bfloat16        pinned
 *   eri_oracle_nearest_index   brute-force argmin over 256 entries, round trip      pinned
 *   eri_oracle_hyper_pack      closed forms at t = 1, f64 restatement               pinned
 *   eri_oracle_step_tensor     closed forms (zero grad, first step), torch.optim.Adam with the
 *                              quantiser bypassed, block-max brute force, and bit-for-bit
 *                              agreement with the independent NumPy restatement
 *                              (oracle/adam8_numpy.py)                              pinned
 *   mode BNB of the step       with wd = 0 it IS torch.optim.Adam's formula (denominator
 *                              sqrt(v)/sqrt(bc2) + eps): 60 steps against torch.optim.Adam;
 *                              decay factor and sign rule by closed form.  Bit-level equality
 *                              with bitsandbytes itself (its fast division, its
 *                              quantisation search)                                  parity unpinned
 *   eri_oracle_adamw32_step    closed form at step 1, float64 recurrence, the reference's
 *                              own 2x2 test case                                     pinned
 *   eri_oracle_adamw32_step_scaled   equals the unscaled step on pre-multiplied fp32
 *                              gradients                                             pinned
 *   eri_oracle_ema_update      float64 closed form; bf16 intermediate rounding of flame-core
 *                              unknown                                               parity unpinned (bf16)
 *   bit-level equality with the reference's own legacy per-tensor linear format
 *   (adam8bit.rs:211-241, flame-core's to_dtype(U8)/round semantics are absent)     parity unpinned
 *
 * The bias corrections of mode L2 are 1 - beta^s with an integer s; the reference forms the power with Rust's
 * f64::powi (adam8bit.rs:164-175), this file with C's pow(beta, (double)s).  Both are f64 results that are
 * then rounded to f32, but powi multiplies repeatedly while pow is correctly rounded, so the two can differ in
 * the last f64 bit before that cast, and in rare cases in the last f32 bit after it.  A wrong exponent or base
 * would show at once (closed forms at steps 2, 7 and 40); that last bit cannot be pinned without a Rust
 * toolchain.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off, no fast-math: every fp32 operation
 * below must round exactly once).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ERI_ORACLE_BLOCK 2048

enum { ERI_ORACLE_MODE_ERI = 0, ERI_ORACLE_MODE_L2 = 1, ERI_ORACLE_MODE_BNB = 2 };
enum { ERI_ORACLE_F32 = 0, ERI_ORACLE_BF16 = 2 };

typedef struct EriOracleHyper {
    float beta1;        /* (float)beta1                                   adam8bit_enhanced.rs:256 */
    float beta2;        /* (float)beta2                                   :260 */
    float omb1;         /* ERI: 1.0f - (float)beta1 (fp32 subtraction)    :256
                           L2 : (float)(1.0 - beta1)  (f64 subtraction)   adam8bit.rs:142 */
    float omb2;         /* same for beta2                                 :260 / adam8bit.rs:151 */
    float eps;          /* (float)eps                                     :263 / adam8bit.rs:186
                           BNB: (float)(eps * sqrt(bc2)) */
    float weight_decay; /* (float)wd                                      :268 / adam8bit.rs:117
                           BNB: the decay factor (float)(1 - lr*wd) */
    float step_size;    /* ERI: (float)(lr*sqrt(bc2)/bc1)                 :213-215,:274
                           L2 : (float)lr                                 adam8bit.rs:193 */
    float bc1;          /* L2 : (float)(1 - beta1^s), s = max(step,1)     adam8bit.rs:164-168 */
    float bc2;          /* L2 : (float)(1 - beta2^s)                      adam8bit.rs:175 */
    float grad_scale;   /* multiplies every gradient first (clip factor / per-layer LR multiplier,
                           pipeline_flux_lora_sequential.rs:759-766,1198-1213); 1.0f = off */
    int32_t mode;
    int32_t use_grad_scale;
} EriOracleHyper;

/* ---- bf16 <-> fp32 -------------------------------------------------------------------- */

float eri_oracle_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

/* round-to-nearest-even; NaN stays NaN (quiet bit forced) */
uint16_t eri_oracle_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* ---- quantiser ------------------------------------------------------------------------ */

/* mid[j] = (map[j] + map[j+1]) * 0.5f, j = 0..254, in fp32 */
void eri_oracle_midpoints(const float *map, float *mid) {
    for (int j = 0; j < 255; ++j) {
        float s = map[j] + map[j + 1];
        mid[j] = s * 0.5f;
    }
}

/* Number of midpoints strictly below x: the nearest map entry, the lower index on an exact tie.
 * NaN compares false everywhere and lands on code 0. */
int eri_oracle_nearest_index(const float *mid, float x) {
    int lo = 0, hi = 255; /* answer in [lo, hi] */
    while (lo < hi) {
        int c = (lo + hi) >> 1;
        if (x > mid[c]) lo = c + 1; else hi = c;
    }
    return lo;
}

/* ---- per-step scalars ----------------------------------------------------------------- */

/* step = the optimizer's counter AFTER its increment for ERI (adam8bit_enhanced.rs:203), the
 * counter as it stands when update() is called for L2 (adam8bit.rs:164, bumped later by step()). */
void eri_oracle_hyper_pack(double lr, double beta1, double beta2, double eps, double wd,
                           uint64_t step, int mode, EriOracleHyper *h) {
    memset(h, 0, sizeof(*h));
    h->mode = mode;
    h->beta1 = (float)beta1;
    h->beta2 = (float)beta2;
    h->eps = (float)eps;
    h->weight_decay = (float)wd;
    h->grad_scale = 1.0f;
    h->use_grad_scale = 0;
    if (mode == ERI_ORACLE_MODE_L2) {
        uint64_t s = step < 1 ? 1 : step;
        h->omb1 = (float)(1.0 - beta1);
        h->omb2 = (float)(1.0 - beta2);
        h->bc1 = (float)(1.0 - pow(beta1, (double)(int32_t)s));
        h->bc2 = (float)(1.0 - pow(beta2, (double)(int32_t)s));
        h->step_size = (float)lr;
    } else {
        double t = (double)step;
        double bc1 = 1.0 - pow(beta1, t);
        double bc2 = 1.0 - pow(beta2, t);
        h->omb1 = 1.0f - h->beta1;
        h->omb2 = 1.0f - h->beta2;
        h->bc1 = (float)bc1;
        h->bc2 = (float)bc2;
        h->step_size = (float)(lr * (sqrt(bc2) / bc1));
        if (mode == ERI_ORACLE_MODE_BNB) {
            h->eps = (float)(eps * sqrt(bc2));
            h->weight_decay = (float)(1.0 - lr * wd);
        }
    }
}

/* ---- one block ------------------------------------------------------------------------ */

static inline float load_elem(const void *base, uint64_t i, int dtype) {
    if (dtype == ERI_ORACLE_F32) return ((const float *)base)[i];
    return eri_oracle_bf16_to_f32(((const uint16_t *)base)[i]);
}

static void step_block(void *p, const void *g, uint8_t *mc, uint8_t *vc, float *am, float *av,
                       uint64_t base, int n, int dtype, int g_dtype, const EriOracleHyper *h,
                       const float *map_s, const float *map_u, const float *mid_s,
                       const float *mid_u) {
    float mbuf[ERI_ORACLE_BLOCK], vbuf[ERI_ORACLE_BLOCK];
    const float a_m = *am, a_v = *av;
    float new_am = 0.0f, new_av = 0.0f;
    for (int i = 0; i < n; ++i) {
        const uint64_t e = base + (uint64_t)i;
        float m_old = map_s[mc[e]] * a_m;
        float v_old = map_u[vc[e]] * a_v;
        float gr = load_elem(g, e, g_dtype);            /* the gradient as F32, whatever it is stored in: :231-235 */
        float pf = load_elem(p, e, dtype);
        if (h->use_grad_scale) gr = gr * h->grad_scale;
        if (h->mode == ERI_ORACLE_MODE_L2 && h->weight_decay > 0.0f) {
            float pw = pf * h->weight_decay;            /* adam8bit.rs:113-120 */
            gr = gr + pw;
        }
        float t1 = m_old * h->beta1;                    /* adam8bit_enhanced.rs:256 */
        float t2 = gr * h->omb1;
        float m = t1 + t2;
        float gg = gr * gr;                             /* :259 */
        float t3 = v_old * h->beta2;                    /* :260 */
        float t4 = gg * h->omb2;
        float v = t3 + t4;
        mbuf[i] = m;
        vbuf[i] = v;
        new_am = fmaxf(new_am, fabsf(m));
        new_av = fmaxf(new_av, fabsf(v));

        float pn;
        if (h->mode == ERI_ORACLE_MODE_L2) {
            float mh = m / h->bc1;                      /* adam8bit.rs:170 */
            float vh = v / h->bc2;                      /* :178 */
            vh = fmaxf(vh, 0.0f);                       /* :181-182 */
            float den = sqrtf(vh) + h->eps;             /* :187 */
            float upd = mh / den;
            float us = upd * h->step_size;              /* :196 */
            if (dtype == ERI_ORACLE_BF16)               /* :197-198 update cast to the param dtype */
                us = eri_oracle_bf16_to_f32(eri_oracle_f32_to_bf16(us));
            pn = pf - us;                               /* :205 */
        } else if (h->mode == ERI_ORACLE_MODE_BNB) {
            float den = sqrtf(v) + h->eps;              /* eps already times sqrt(bc2) */
            float r = m / den;
            float us = r * h->step_size;
            pn = pf - us;
            if (h->weight_decay != 1.0f) pn = pn * h->weight_decay; /* decay factor, after the Adam term */
        } else {
            float den = sqrtf(v) + h->eps;              /* adam8bit_enhanced.rs:263 */
            float r = m / den;                          /* :264 */
            float u = r;
            if (h->weight_decay > 0.0f) {               /* :267-271 */
                float pw = pf * h->weight_decay;
                u = r + pw;
            }
            float us = u * h->step_size;                /* :274 */
            pn = pf - us;                               /* :275 apply_update: p <- p - x */
        }
        if (dtype == ERI_ORACLE_F32) ((float *)p)[e] = pn;
        else ((uint16_t *)p)[e] = eri_oracle_f32_to_bf16(pn);
    }
    for (int i = 0; i < n; ++i) {
        const uint64_t e = base + (uint64_t)i;
        float xm = (new_am == 0.0f) ? 0.0f : mbuf[i] / new_am;
        float xv = (new_av == 0.0f) ? 0.0f : vbuf[i] / new_av;
        int cm = eri_oracle_nearest_index(mid_s, xm);
        if (h->mode == ERI_ORACLE_MODE_BNB && new_am != 0.0f && isfinite(mbuf[i]) &&
            (signbit(map_s[cm]) != 0) != (signbit(mbuf[i]) != 0)) {
            if (mbuf[i] > 0.0f) cm += 1; else cm -= 1; /* keep the sign of the first moment */
        }
        mc[e] = (uint8_t)cm;
        vc[e] = (uint8_t)eri_oracle_nearest_index(mid_u, xv);
    }
    *am = new_am;
    *av = new_av;
}

/*
 * One step over one tensor.  Returns 0, or -1 for an empty tensor (the reference refuses to
 * quantise an empty tensor, adam8bit_enhanced.rs:46-50), -2 for an unsupported dtype.
 * threads <= 1 runs serially; otherwise blocks are split statically over that many threads.
 */
/* `g_dtype` is the storage type of the gradient, which may differ from the parameter's: the reference
 * casts every gradient to F32 before it uses it and never rounds it back
 * (adam8bit_enhanced.rs:231-235, adam8bit.rs:110). */
int eri_oracle_step_tensor_g(void *p, const void *g, uint8_t *m, uint8_t *v, float *absmax_m,
                             float *absmax_v, uint64_t numel, int dtype, int g_dtype, const EriOracleHyper *h,
                             const float *map_s, const float *map_u, int threads) {
    if (numel == 0) return -1;
    if (dtype != ERI_ORACLE_F32 && dtype != ERI_ORACLE_BF16) return -2;
    if (g_dtype != ERI_ORACLE_F32 && g_dtype != ERI_ORACLE_BF16) return -2;
    float mid_s[255], mid_u[255];
    eri_oracle_midpoints(map_s, mid_s);
    eri_oracle_midpoints(map_u, mid_u);
    const int64_t nblocks = (int64_t)((numel + ERI_ORACLE_BLOCK - 1) / ERI_ORACLE_BLOCK);
    (void)threads;
#ifdef _OPENMP
#pragma omp parallel for schedule(static) num_threads(threads > 1 ? threads : 1)
#endif
    for (int64_t b = 0; b < nblocks; ++b) {
        uint64_t base = (uint64_t)b * ERI_ORACLE_BLOCK;
        uint64_t left = numel - base;
        int n = left < ERI_ORACLE_BLOCK ? (int)left : ERI_ORACLE_BLOCK;
        step_block(p, g, m, v, absmax_m + b, absmax_v + b, base, n, dtype, g_dtype, h, map_s, map_u, mid_s,
                   mid_u);
    }
    return 0;
}

/* Gradient stored in the parameter's dtype. */
int eri_oracle_step_tensor(void *p, const void *g, uint8_t *m, uint8_t *v, float *absmax_m,
                           float *absmax_v, uint64_t numel, int dtype, const EriOracleHyper *h,
                           const float *map_s, const float *map_u, int threads) {
    return eri_oracle_step_tensor_g(p, g, m, v, absmax_m, absmax_v, numel, dtype, dtype, h, map_s, map_u, threads);
}

/* Fresh state: the codes of 0.0 with absmax 0, what quantising a zeros tensor gives
 * (the reference initialises from Tensor::zeros, adam8bit_enhanced.rs:179-197). */
void eri_oracle_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v,
                           uint64_t numel) {
    uint64_t nblocks = (numel + ERI_ORACLE_BLOCK - 1) / ERI_ORACLE_BLOCK;
    memset(m, 127, numel);
    memset(v, 0, numel);
    for (uint64_t b = 0; b < nblocks; ++b) { absmax_m[b] = 0.0f; absmax_v[b] = 0.0f; }
}

/* Blockwise dequantisation of a state to fp32 (checkpoint export, adam8bit.rs:296-308). */
void eri_oracle_dequantize(const uint8_t *codes, const float *absmax, const float *map,
                           uint64_t numel, float *out) {
    for (uint64_t i = 0; i < numel; ++i) out[i] = map[codes[i]] * absmax[i / ERI_ORACLE_BLOCK];
}

/* Blockwise quantisation of an fp32 tensor (checkpoint import, adam8bit.rs:316-329). */
void eri_oracle_quantize(const float *x, const float *map, uint64_t numel, uint8_t *codes,
                         float *absmax) {
    float mid[255];
    eri_oracle_midpoints(map, mid);
    uint64_t nblocks = (numel + ERI_ORACLE_BLOCK - 1) / ERI_ORACLE_BLOCK;
    for (uint64_t b = 0; b < nblocks; ++b) {
        uint64_t base = b * ERI_ORACLE_BLOCK;
        uint64_t n = numel - base < ERI_ORACLE_BLOCK ? numel - base : ERI_ORACLE_BLOCK;
        float a = 0.0f;
        for (uint64_t i = 0; i < n; ++i) a = fmaxf(a, fabsf(x[base + i]));
        for (uint64_t i = 0; i < n; ++i) {
            float q = (a == 0.0f) ? 0.0f : x[base + i] / a;
            codes[base + i] = (uint8_t)eri_oracle_nearest_index(mid, q);
        }
        absmax[b] = a;
    }
}

/* ---- 32-bit sibling and EMA ------------------------------------------------------------------ */

/* AdamW::step_with_grads, crates/common/optim/src/adamw.rs:20-58: fp32 math on fp32 moments, no bias
 * correction, decoupled decay, parameter cast back to its dtype.  Pinned by closed forms at the
 * first step, a float64 recurrence and the reference's own test case (2x2 bf16 ones, grad ones,
 * src/tests/adamw_step.rs:6-30). */
/* master != NULL: mixed precision (src/kernels/fused_adam.cu:151-193): the fp32 master copy is the value
 * that is read and updated, and p receives its rounded value.  Pinned by: the master after any number
 * of steps equals what the fp32 path gives on the same gradients, and p equals the rounded master. */
static void adamw32_step(void *p, const void *g, float *m, float *v, uint64_t numel, int dtype, float lr,
                         float beta1, float beta2, float eps, float wd, float *master, int scaled, float gscale) {
    const float omb1 = 1.0f - beta1, omb2 = 1.0f - beta2, neg_lr = -lr;
    for (uint64_t i = 0; i < numel; ++i) {
        float pf = master ? master[i] : load_elem(p, i, dtype), gr = load_elem(g, i, dtype);
        if (scaled) gr = gr * gscale; /* one rounded product, as in the 8-bit step (step_elem above) */
        float ms = m[i] * beta1;       /* :35 */
        float gs = gr * omb1;          /* :36 */
        float mn = ms + gs;            /* :37 */
        float vs = v[i] * beta2;       /* :40 */
        float g2 = gr * gr;            /* :41 */
        float g2s = g2 * omb2;         /* :42 */
        float vn = vs + g2s;           /* :43 */
        float denom = sqrtf(vn) + eps; /* :46 */
        float update = mn / denom;     /* :47 */
        float w = wd != 0.0f ? pf * wd : 0.0f; /* :50 */
        float total = update + w;      /* :51 */
        float step = total * neg_lr;   /* :52 */
        float pn = pf + step;
        m[i] = mn;
        v[i] = vn;
        if (master) master[i] = pn;
        if (dtype == ERI_ORACLE_F32) ((float *)p)[i] = pn;
        else ((uint16_t *)p)[i] = eri_oracle_f32_to_bf16(pn); /* :55 */
    }
}

void eri_oracle_adamw32_step(void *p, const void *g, float *m, float *v, uint64_t numel, int dtype, float lr,
                             float beta1, float beta2, float eps, float wd, float *master) {
    adamw32_step(p, g, m, v, numel, dtype, lr, beta1, beta2, eps, wd, master, 0, 1.0f);
}

/* The same step on gradients multiplied by `gscale` first: the clip factor of the global norm and the loss-scale
 * and per-layer multipliers, which the reference applies by rewriting the gradients before the optimizer runs
 * (clip_gradients, pipeline_flux_lora_sequential.rs:1198-1213; pipeline_flux_lora_1024.rs:691-697).  Pinned by:
 * equals the unscaled step on gradients multiplied beforehand (fp32 tensors, where that product is not rounded
 * to the tensor's dtype in between). */
void eri_oracle_adamw32_step_scaled(void *p, const void *g, float *m, float *v, uint64_t numel, int dtype, float lr,
                                    float beta1, float beta2, float eps, float wd, float *master, float gscale) {
    adamw32_step(p, g, m, v, numel, dtype, lr, beta1, beta2, eps, wd, master, 1, gscale);
}

/* EMA update, src/trainers/ema_enhanced.rs:91-100: shadow = shadow*decay + p*(1 - decay) in fp32,
 * cast to the tensors' dtype.  Whether flame-core rounds the two products to bf16 first for bf16
 * tensors cannot be read from the tree: parity unpinned for that detail. */
void eri_oracle_ema_update(void *shadow, const void *p, uint64_t numel, int dtype, float decay) {
    const float omd = 1.0f - decay;
    for (uint64_t i = 0; i < numel; ++i) {
        float a = load_elem(shadow, i, dtype) * decay;
        float b = load_elem(p, i, dtype) * omd;
        float s = a + b;
        if (dtype == ERI_ORACLE_F32) ((float *)shadow)[i] = s;
        else ((uint16_t *)shadow)[i] = eri_oracle_f32_to_bf16(s);
    }
}

int eri_oracle_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
