/*
 * The plain step kernel (one wave per block, no cross-block prefetch): large tables of fp32 parameters and
 * of bf16 parameters with fp32 gradients, bf16 tables in the functional update's arithmetic, and any table
 * with ERI_ADAM8_FLAG_BSEARCH, ERI_ADAM8_FLAG_NO_PIPELINE or ERI_ADAM8_FLAG_ONE_WAVE.  Compiled twice,
 * once per parameter dtype (-DERI_PLAIN_BF16=0|1), so that the two halves build in parallel.
 */
#include "eri_adam8_inline.h"

#ifndef ERI_PLAIN_BF16
#error "compile with -DERI_PLAIN_BF16=0 or 1"
#endif


namespace eri {

/* Threads per workgroup: sixteen waves per compute unit where the instantiation fits the 128 registers that
 * leaves each lane, twelve (170 registers) where it would spill: the coupled-decay mode with a gradient scale,
 * with fp32 gradients or with the binary search (12-30 spilled registers at sixteen waves). */
constexpr uint32_t plain_threads(int mode, bool gs, bool keytab, bool gbf16) {
    return (mode == ERI_ADAM8_MODE_L2 && (gs || !keytab || !gbf16)) ? 768 : 1024;
}

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB, bool GBF16>
__global__ __launch_bounds__(plain_threads(MODE, GS, KEYTAB, GBF16)) void adam8_step_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                          uint32_t total_blocks, EriAdam8Hyper h_in,
                                                          const uint4 *__restrict__ lds_image,
                                                          const float *__restrict__ dev_scale) {
    ERI_LDS_IMAGE;
    __shared__ float decayed[16][2][256]; // per wave: the values its block's state codes stand for, decayed
    const StepHyper h = make_step_hyper<MODE>(h_in);
    // clip factor left on the device by the gradient-norm pass (1.0 when there is none)
    const float tscale = (GS && dev_scale) ? *dev_scale : 1.0f;
    // the binary search needs the maps and midpoints only (4 KB); the slot tables are the other 96 KB
    constexpr uint32_t staged = KEYTAB ? kLdsImageBytes : kOffKeyU;
    for (uint32_t i = threadIdx.x; i < staged / 16; i += blockDim.x) lds_raw[i] = lds_image[i];
    __syncthreads();
    const char *base = reinterpret_cast<const char *>(lds_raw);
    Lds L;
    L.map_s = reinterpret_cast<const float *>(base + kOffMapS);
    L.map_u = reinterpret_cast<const float *>(base + kOffMapU);
    L.mid_s = reinterpret_cast<const float *>(base + kOffMidS);
    L.mid_u = reinterpret_cast<const float *>(base + kOffMidU);
    L.key_s = base + kOffKeyS;
    L.key_u = base + kOffKeyU;

    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    const uint32_t stride = gridDim.x * waves_per_wg;
    const BlockDiv dbc1(h.bc1), dbc2(h.bc2);

    // Full blocks: round k gives wave w block k * stride + w, and the blocks left over when the list does not
    // divide (fewer than one per wave) go one to each workgroup in turn -- workgroup i takes left-over blocks
    // i, i + grid, i + 2 grid, ... on its first waves -- so that the short last round runs on every compute
    // unit instead of filling the first few (2-3 % of the launch on tables of 5-20 blocks per wave).
    const uint32_t wave_in_wg = threadIdx.x / kWave;
    const uint32_t rounds = total_blocks / stride;
    const uint32_t left_first = rounds * stride;
    const uint32_t left_mine = wave_in_wg * gridDim.x + blockIdx.x;
    const bool has_left = left_first + left_mine < total_blocks;

    // partial last blocks first: one per row at most, one to each workgroup in turn, from a workgroup's last
    // wave backwards: those are the waves without a left-over block, so the slower element-wise tail lands
    // where there is slack
    for (uint32_t r = blockIdx.x + (waves_per_wg - 1 - wave_in_wg) * gridDim.x; r < n_rows; r += stride) {
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        if (n != 0) {
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            tail_block<BF16, MODE, EXACT, WD, GS, KEYTAB, GBF16>(t, (uint32_t)(t.numel / kBlock), n, lane, h, gscale, dbc1, dbc2, L);
        }
    }
    uint32_t ti = 0, t_end = 0;
    DevTensor t;
    const BlockRowMap map(rows, n_rows);
    const uint32_t trips = rounds + (has_left ? 1u : 0u);
    for (uint32_t k = 0; k < trips; ++k) {
        const uint32_t blk = k < rounds ? k * stride + wave : left_first + left_mine;
        map.seek(rows, blk, ti, t, t_end);
        const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
        full_block<BF16, MODE, EXACT, WD, GS, KEYTAB, GBF16>(t, blk - t.full_start, lane, h, gscale, dbc1, dbc2, L,
                                                             decayed[threadIdx.x / kWave]);
    }
}

namespace {

constexpr bool kBf16 = ERI_PLAIN_BF16 != 0;

template <int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB, bool GBF16>
int launch_one(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
               const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    auto k = adam8_step_kernel<kBf16, MODE, EXACT, WD, GS, KEYTAB, GBF16>;
    if (wg > plain_threads(MODE, GS, KEYTAB, GBF16)) wg = plain_threads(MODE, GS, KEYTAB, GBF16);
    // One common window for all dies (a grid-stride walk): on the tables this kernel takes, up to 1,024
    // blocks per compute unit, it measured 2 % ahead of one range per die with the arrays far apart in device
    // memory and 5 % with them adjacent; the tables of the prefetching kernel want the ranges.
    hipLaunchKernelGGL(k, dim3(grid), dim3(wg), 0, s, rows, n_rows, total_blocks, h,
                       static_cast<const uint4 *>(lds_image), dev_scale);
    return (int)hipGetLastError();
}

/* BSEARCH selects the cross-check variants (binary search of the midpoint table); mode BNB has none. */
template <int MODE, bool EXACT, bool BSEARCH, bool GBF16 = kBf16>
int launch_flags(bool wd, bool gs, bool keytab, const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks,
                 const EriAdam8Hyper &h, const void *img, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
#define ERI_GO(W, G, K) return launch_one<MODE, EXACT, W, G, K, GBF16>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s)
    if (BSEARCH && !keytab) {
        if (wd) { if (gs) ERI_GO(true, true, !BSEARCH); ERI_GO(true, false, !BSEARCH); }
        if (gs) ERI_GO(false, true, !BSEARCH);
        ERI_GO(false, false, !BSEARCH);
    }
    if (wd) { if (gs) ERI_GO(true, true, true); ERI_GO(true, false, true); }
    if (gs) ERI_GO(false, true, true);
    ERI_GO(false, false, true);
#undef ERI_GO
}

} // namespace

#if ERI_PLAIN_BF16
int launch_step_plain_bf16(int mode, bool exact, bool wd, bool gs, bool keytab, bool grad_f32, const DevTensor *rows,
                           uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h, const void *img,
                           const float *dev_scale, uint32_t grid, uint32_t wg, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
#define ERI_ARGS wd, gs, keytab, rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s
    if (grad_f32) { // fp32 gradients for bf16 parameters: slot-table variants only
        if (!keytab) return (int)hipErrorInvalidValue;
        if (mode == ERI_ADAM8_MODE_BNB)
            return exact ? launch_flags<ERI_ADAM8_MODE_BNB, true, false, false>(ERI_ARGS)
                         : launch_flags<ERI_ADAM8_MODE_BNB, false, false, false>(ERI_ARGS);
        if (mode == ERI_ADAM8_MODE_L2) return launch_flags<ERI_ADAM8_MODE_L2, true, false, false>(ERI_ARGS);
        return exact ? launch_flags<ERI_ADAM8_MODE_ERI, true, false, false>(ERI_ARGS)
                     : launch_flags<ERI_ADAM8_MODE_ERI, false, false, false>(ERI_ARGS);
    }
    if (mode == ERI_ADAM8_MODE_BNB)
        return exact ? launch_flags<ERI_ADAM8_MODE_BNB, true, false>(ERI_ARGS) : launch_flags<ERI_ADAM8_MODE_BNB, false, false>(ERI_ARGS);
    if (mode == ERI_ADAM8_MODE_L2) return launch_flags<ERI_ADAM8_MODE_L2, true, true>(ERI_ARGS); // always the IEEE chain
    return exact ? launch_flags<ERI_ADAM8_MODE_ERI, true, true>(ERI_ARGS) : launch_flags<ERI_ADAM8_MODE_ERI, false, true>(ERI_ARGS);
#undef ERI_ARGS
}
#else
/* fp32 parameters always take the IEEE square root and division. */
int launch_step_plain_f32(int mode, bool wd, bool gs, bool keytab, const DevTensor *rows, uint32_t n_rows,
                          uint32_t total_blocks, const EriAdam8Hyper &h, const void *img, const float *dev_scale,
                          uint32_t grid, uint32_t wg, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
#define ERI_ARGS wd, gs, keytab, rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s
    if (mode == ERI_ADAM8_MODE_BNB) return launch_flags<ERI_ADAM8_MODE_BNB, true, false>(ERI_ARGS);
    if (mode == ERI_ADAM8_MODE_L2) return launch_flags<ERI_ADAM8_MODE_L2, true, true>(ERI_ARGS);
    return launch_flags<ERI_ADAM8_MODE_ERI, true, true>(ERI_ARGS);
#undef ERI_ARGS
}
#endif

} // namespace eri
