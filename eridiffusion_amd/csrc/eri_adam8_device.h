/*
 * Layouts shared by the host side of the library and its gfx950 kernels: the device row of the
 * launch table and the image of lookup tables every workgroup stages into LDS.
 */
#ifndef ERI_ADAM8_DEVICE_H
#define ERI_ADAM8_DEVICE_H

#include <stdint.h>

#include "../../include/eri_optim8.h"

namespace eri {

constexpr uint32_t kBlock = ERI_ADAM8_BLOCK; /* elements per quantisation block, one wavefront each */
constexpr uint32_t kWave = 64;

/* One tensor as the kernels see it (80 bytes, read through scalar loads). */
struct DevTensor {
    void *p;          /* new parameters are written here */
    const void *p_in; /* old parameters are read from here: p itself for an in-place update */
    const void *g;
    uint8_t *m;
    uint8_t *v;
    float *absmax_m;
    float *absmax_v;
    uint64_t numel;
    uint32_t full_start;  /* number of full 2048-element blocks in the rows before this one (same dtype) */
    float grad_scale;
    void *shadow;     /* EMA shadow of the parameter, or null */
};
static_assert(sizeof(DevTensor) == 80, "DevTensor must stay 80 bytes");

/* How the elements of one group of rows are stored: parameters and gradients F32, both BF16, or BF16
 * parameters with F32 gradients (the reference casts every gradient to F32 and never rounds it). */
enum Layout { kLayoutF32 = 0, kLayoutBF16 = 1, kLayoutBF16GradF32 = 2, kLayouts = 3 };
inline bool layout_param_bf16(int layout) { return layout != kLayoutF32; }
inline bool layout_grad_bf16(int layout) { return layout == kLayoutBF16; }

/*
 * Requantisation without a search.  The quotient x = value / absmax in [-1, 1] is produced
 * already multiplied by kKeyScale (a power of two, so nothing is rounded differently), converted
 * to binary16 rounded toward zero (both moments in one v_cvt_pkrtz_f16_f32), and the top bits of that half float -- sign, exponent
 * and the leading mantissa bits -- select a slot.  The slots are narrow enough that at most one
 * midpoint of the map lies inside any of them, so
 *     code(x) = slot.lo + (x * kKeyScale > slot.mid)
 * equals the number of midpoints below x, i.e. the binary search's answer, ties included.
 * Every binary16 pattern has a slot: there is nothing to clamp, NaN lands in slots that answer 0
 * (a search finds every comparison false), and the scale keeps all midpoints in the normal
 * binary16 range, so the result does not depend on how half denormals are treated.
 */
struct KeySlot {
    float mid;   /* the one midpoint inside the slot times kKeyScale, +inf if there is none */
    uint32_t lo; /* number of midpoints below every value of the slot */
};

constexpr float kKeyScale = 4096.0f;
constexpr float kKeyScaleInv = 1.0f / 4096.0f;
constexpr uint32_t kSKeyDrop = 4;   /* signed map: keep 6 mantissa bits of the half float */
constexpr uint32_t kUKeyDrop = 3;   /* unsigned map: keep 7 */
constexpr uint32_t kSKeyStride = 16; /* bytes between signed slots: address = half & 0xfff0 */
constexpr uint32_t kUKeyStride = 8;  /* bytes between unsigned slots: address = half & 0x7ff8 */
constexpr uint32_t kSKeyCount = 1u << (16 - kSKeyDrop); /* 4096, sign included */
constexpr uint32_t kUKeyCount = 1u << (15 - kUKeyDrop); /* 4096, sign masked off */

/* Byte offsets inside the LDS image. */
constexpr uint32_t kOffMapS = 0;                              /* 256 floats: code -> value */
constexpr uint32_t kOffMapU = kOffMapS + 1024;                /* 256 floats */
constexpr uint32_t kOffMidS = kOffMapU + 1024;                /* 255 midpoints + one +inf */
constexpr uint32_t kOffMidU = kOffMidS + 1024;
/* Both slot tables start below 64 KiB so that their offsets fit the 16-bit immediate of ds_read. */
constexpr uint32_t kOffKeyU = kOffMidU + 1024;                /* kUKeyCount slots, kUKeyStride apart */
constexpr uint32_t kOffKeyS = kOffKeyU + kUKeyCount * kUKeyStride; /* kSKeyCount slots */
constexpr uint32_t kLdsImageBytes = kOffKeyS + kSKeyCount * kSKeyStride;
static_assert(kOffKeyS < 65536 && kOffKeyU < 65536, "slot table offsets must fit a ds_read immediate");
static_assert(kLdsImageBytes % 16 == 0, "the image is staged in 16-byte words");

/* Launchers implemented in eri_adam8_kernels.hip; `stream` is a hipStream_t.  All return a
 * hipError_t as int.  `lds_image` is the device copy of the kLdsImageBytes table image. */
int launch_step(const DevTensor *rows, uint32_t n_rows, uint32_t total_full_blocks, int layout,
                const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg,
                uint32_t compute_units, void *stream);

constexpr uint32_t kChunks = 8;           /* contiguous ranges the block list is cut into: one per accelerator die */
constexpr uint32_t kSplitBlocksPerCu = 64; /* tables of at most this many full blocks per compute unit take the
                                              four-waves-per-block kernel */
constexpr uint32_t kPrefetchBlocksPerCu = 1024; /* bf16 tables take the prefetching kernel above this many full blocks
                                                   per compute unit; up to it, sixteen waves without a prefetch are
                                                   2-4 % faster than twelve with one (measured at 292-876 per unit,
                                                   the other way round from 1,168) */
constexpr uint32_t kNormWaves = 4;        /* waves per workgroup of the gradient-norm pass */

/* The chunked walk (BlockWalk) needs the same number of workgroups in every chunk. */
inline uint32_t chunks_for(uint32_t grid) { return grid % kChunks == 0 ? kChunks : 1u; }

/* The step's kernels live in translation units of their own (they build in parallel); launch_step
 * picks one.  wd / gs / keytab / exact select template instances: decay present, gradient scale present,
 * slot-table (rather than binary-search) requantisation, IEEE square root and division on bf16. */
int launch_step_plain_f32(int mode, bool wd, bool gs, bool keytab, const DevTensor *rows, uint32_t n_rows,
                          uint32_t total_blocks, const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale,
                          uint32_t grid, uint32_t wg, void *stream);
int launch_step_plain_bf16(int mode, bool exact, bool wd, bool gs, bool keytab, bool grad_f32, const DevTensor *rows, uint32_t n_rows,
                           uint32_t total_blocks, const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale,
                           uint32_t grid, uint32_t wg, void *stream);
/* Four waves per block, for tables of few blocks; `grid` workgroups of 1024 threads. */
int launch_step_split(int layout, int mode, bool exact, bool wd, bool gs, const DevTensor *rows, uint32_t n_rows,
                      uint32_t total_blocks, const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale,
                      uint32_t grid, uint32_t teams, void *stream);
/* Whether launch_step would run this group on the prefetching kernel with the EMA update inside it. */
bool step_fuses_ema(uint32_t total_full_blocks, int layout, const EriAdam8Hyper &h, uint32_t compute_units);
int launch_step_pipelined(int mode, bool exact, bool wd, bool gs, bool ema, const DevTensor *rows, uint32_t n_rows,
                          uint32_t total_blocks, const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale,
                          uint32_t grid, uint32_t wg, void *stream);
/* The same kernel for bf16 parameters whose gradients are fp32. */
int launch_step_pipelined_grad_f32(int mode, bool exact, bool wd, bool gs, bool ema, const DevTensor *rows, uint32_t n_rows,
                                   uint32_t total_blocks, const EriAdam8Hyper &h, const void *lds_image,
                                   const float *dev_scale, uint32_t grid, uint32_t wg, void *stream);
/* The same kernel for fp32 parameters (IEEE chain throughout, no EMA inside it). */
int launch_step_pipelined_f32(int mode, bool wd, bool gs, const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks,
                              const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, uint32_t grid,
                              uint32_t wg, void *stream);
/* Sum of |moment - dequantised moment| of the coming step, per row: err[2r] first moment, err[2r+1] second. */
int launch_quant_error(const DevTensor *rows, uint32_t n_rows, uint32_t total_full_blocks, int layout,
                       const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, double *err,
                       uint32_t grid, void *stream);
/* Gradient norm: one f64 partial per wave (grid * 4 of them), then norm and clip factor into out[0], out[1]. */
constexpr uint32_t kNormWavesPerCu = 32; // persistent waves of the gradient-norm pass per compute unit
int launch_grad_sumsq(const DevTensor *rows, uint32_t n_rows, uint32_t total_full_blocks, bool grad_bf16,
                      double *partial, uint32_t grid, void *stream);
int launch_grad_norm_finish(const double *partial, uint32_t n, float max_norm, float denom_eps, float *out,
                            void *stream);
/* Diagnostics: reads and rewrites (unchanged) every full block of a group of bf16 rows as the step does. */
int launch_traffic_probe(const DevTensor *rows, uint32_t n_rows, uint32_t total_full_blocks, uint32_t grid, void *stream);
/* Clears `bytes` bytes at `p`; both multiples of 16. */
int launch_fill_zero(void *p, size_t bytes, void *stream);
int launch_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel, void *stream);
int launch_dequantize(const uint8_t *codes, const float *absmax, int signed_map, uint64_t numel, float *out,
                      const void *lds_image, void *stream);
int launch_quantize(const float *x, int signed_map, uint64_t numel, uint8_t *codes, float *absmax,
                    const void *lds_image, void *stream);

/* Row of the plain element-wise sweeps (32-bit AdamW, EMA): up to five streams of one tensor. */
struct ElemRow {
    void *a;        /* AdamW: p      EMA: shadow */
    const void *b;  /* AdamW: g      EMA: p */
    void *c;        /* AdamW: m (fp32) */
    void *d;        /* AdamW: v (fp32) */
    void *e;        /* AdamW: fp32 master copy of p, or null */
    uint64_t numel;
    uint32_t full_start; /* full 2048-element blocks in the rows before this one */
    float scale;         /* AdamW: per-layer multiplier of the gradients (used by the scaled step only) */
};
static_assert(sizeof(ElemRow) == 56, "ElemRow must stay 56 bytes");

/* scaled: every gradient is first multiplied by (grad_scale * row.scale) * (*dev_scale, 1 if null), as the 8-bit
 * step does with ERI_ADAM8_FLAG_GRAD_SCALE. */
int launch_adamw32(const ElemRow *rows, uint32_t n_rows, uint32_t total_full_blocks, int dtype_tag,
                   const EriAdamW32Hyper &h, bool scaled, float grad_scale, const float *dev_scale, uint32_t grid,
                   void *stream);
int launch_ema(const ElemRow *rows, uint32_t n_rows, uint32_t total_full_blocks, int dtype_tag, float decay,
               uint32_t grid, void *stream);

} // namespace eri
#endif
