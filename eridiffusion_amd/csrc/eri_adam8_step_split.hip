/*
 * Step kernel for small launch tables: four wavefronts share one 2048-element block.
 *
 * The persistent kernels give every wave a whole block, which is the right shape when there are
 * thousands of blocks per wave-slot of the chip.  A table of a few hundred blocks (one flat tensor of a
 * million parameters, a small adapter) leaves most of the chip idle that way and the launch lasts as long
 * as one wave's trip through one block.  Here a block is cut into four 512-element quarters, one per
 * wave; the block's absmax is the maximum of the four wave maxima (DPP inside the wave, then four floats
 * through LDS and one workgroup barrier), after which every wave requantises its own quarter.  A
 * workgroup is four such teams (1024 threads), so the table image is staged into LDS once per four blocks;
 * a table with fewer blocks than four per compute unit uses `teams` < 4 of them, in more workgroups.
 * Arithmetic, rounding and results are those of the other two kernels.
 */
#include "eri_adam8_inline.h"

namespace eri {

template <bool BF16, bool GBF16, int MODE, bool EXACT, bool WD, bool GS>
__global__ __launch_bounds__(1024) void adam8_step_split_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                                uint32_t total_blocks, EriAdam8Hyper h_in,
                                                                const uint4 *__restrict__ lds_image,
                                                                const float *__restrict__ dev_scale, uint32_t teams) {
    ERI_LDS_IMAGE;
    const StepHyper h = make_step_hyper<MODE>(h_in);
    __shared__ float wave_maxima[2][4][8]; // [parity of the iteration][team][4 x first, 4 x second moment]
    // per wave: (MAP[c] * absmax) * beta for the 2 x 256 codes of the block at hand, formed once per code
    // (8 multiplications per lane) instead of once per element (16 per lane)
    __shared__ float decayed[16][2][256];
    const float tscale = (GS && dev_scale) ? *dev_scale : 1.0f;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
    const uint32_t team = wave_in_wg >> 2;   // 0..3
    const uint32_t quarter = wave_in_wg & 3; // which 512 elements of the team's block
    const uint32_t o = quarter * 512 + lane * 8;

    // One quarter block as it comes from memory.  The first one is requested before the table image is
    // staged, so that its trip to HBM overlaps the staging.
    struct Quarter {
        DevTensor t;
        uint32_t lb;
        bool active;
        Raw8<BF16> pr;
        Raw8<GBF16> gr;
        u32x2 mr, vr;
        float a_m, a_v;
    } q;
    uint32_t ti = 0, t_end = 0;
    const BlockRowMap map(rows, n_rows);
    auto request = [&](uint32_t first) {
        const uint32_t blk = first + team;
        q.active = team < teams && blk < total_blocks;
        if (!q.active) return;
        map.seek(rows, blk, ti, q.t, t_end);
        q.lb = blk - q.t.full_start;
        const size_t e0 = (size_t)q.lb * kBlock;
        const size_t esz = BF16 ? 2 : 4;
        q.pr.load(static_cast<const char *>(q.t.p_in) + e0 * esz, o);
        q.gr.load(static_cast<const char *>(q.t.g) + e0 * (GBF16 ? 2 : 4), o);
        q.mr = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x2 *>(q.t.m + e0 + o)));
        q.vr = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x2 *>(q.t.v + e0 + o)));
        q.a_m = as_global(q.t.absmax_m)[q.lb];
        q.a_v = as_global(q.t.absmax_v)[q.lb];
    };
    request(blockIdx.x * teams);

    for (uint32_t i = threadIdx.x; i < kLdsImageBytes / 16; i += blockDim.x) lds_raw[i] = lds_image[i];
    __syncthreads();
    const char *base = reinterpret_cast<const char *>(lds_raw);
    Lds L;
    L.map_s = reinterpret_cast<const float *>(base + kOffMapS);
    L.map_u = reinterpret_cast<const float *>(base + kOffMapU);
    L.mid_s = reinterpret_cast<const float *>(base + kOffMidS);
    L.mid_u = reinterpret_cast<const float *>(base + kOffMidU);
    L.key_s = base + kOffKeyS;
    L.key_u = base + kOffKeyU;
    const BlockDiv dbc1(h.bc1), dbc2(h.bc2);
    float(*const mine)[256] = decayed[wave_in_wg];
    const f32x4 base_s = reinterpret_cast<const f32x4 *>(L.map_s)[lane]; // codes 4*lane .. 4*lane + 3
    const f32x4 base_u = reinterpret_cast<const f32x4 *>(L.map_u)[lane];

    // partial last blocks: one wave each, no barrier involved
    const uint32_t n_waves = gridDim.x * 16;
    for (uint32_t r = blockIdx.x * 16 + wave_in_wg; r < n_rows; r += n_waves) {
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        if (n != 0) {
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            tail_block<BF16, MODE, EXACT, WD, GS, true, GBF16>(t, (uint32_t)(t.numel / kBlock), n, lane, h, gscale, dbc1, dbc2, L);
        }
    }

    uint32_t parity = 0;
    // every wave of the workgroup runs the same number of iterations: the barrier is inside the loop
    for (uint32_t first = blockIdx.x * teams; first < total_blocks; first += gridDim.x * teams, parity ^= 1) {
        float m[8], v[8];
        float nam = 0.0f, nav = 0.0f;
        // the quarter at hand; q itself is handed to the next request as soon as its raw words are used up
        const bool active = q.active;
        const DevTensor t = q.t;
        const uint32_t lb = q.lb;
        if (active) {
            const size_t e0 = (size_t)lb * kBlock;
            char *p = static_cast<char *>(t.p) + e0 * (BF16 ? 2 : 4);
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            float pv[8], gv[8], pn[8];
            q.pr.unpack(pv);
            q.gr.unpack(gv);
            {
                f32x4 ds, du;
                ds.x = (base_s.x * q.a_m) * h.beta1; ds.y = (base_s.y * q.a_m) * h.beta1;
                ds.z = (base_s.z * q.a_m) * h.beta1; ds.w = (base_s.w * q.a_m) * h.beta1;
                du.x = (base_u.x * q.a_v) * h.beta2; du.y = (base_u.y * q.a_v) * h.beta2;
                du.z = (base_u.z * q.a_v) * h.beta2; du.w = (base_u.w * q.a_v) * h.beta2;
                reinterpret_cast<f32x4 *>(mine[0])[lane] = ds;
                reinterpret_cast<f32x4 *>(mine[1])[lane] = du;
            }
            Redo8 redo; // per element: the exact chain runs for the flagged positions only
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float t1 = lds_float_at(mine[0], code_offset(q.mr, k));
                const float t3 = lds_float_at(mine[1], code_offset(q.vr, k));
                uint64_t flagged = 0;
                adam_elem_decayed<MODE, EXACT, BF16, WD, GS>(pv[k], gv[k], t1, t3, h, gscale, dbc1, dbc2, m[k], v[k], pn[k], flagged);
                redo.set(k, flagged);
                nam = fmaxf(nam, __builtin_fabsf(m[k]));
                nav = fmaxf(nav, __builtin_fabsf(v[k]));
            }
            if (BF16 && MODE == ERI_ADAM8_MODE_L2 && h.l2_all_exact) redo.set_all();
            if (BF16 && redo.any) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (redo.lanes[k] && redo.mine(k)) pn[k] = param_exact<MODE, WD, BF16>(pv[k], m[k], v[k], h, dbc1, dbc2);
            }
            store8<BF16>(p, o, pn);
            wave_max2(nam, nav);
            if (lane == 0) {
                wave_maxima[parity][team][quarter] = nam;
                wave_maxima[parity][team][4 + quarter] = nav;
            }
        }
        __syncthreads();
        // the next quarter's loads travel while this one is requantised
        const uint32_t next = first + gridDim.x * teams;
        if (next < total_blocks) request(next);
        else q.active = false;
        if (active) {
            const float *wm = wave_maxima[parity][team];
            nam = fmaxf(fmaxf(wm[0], wm[1]), fmaxf(wm[2], wm[3]));
            nav = fmaxf(fmaxf(wm[4], wm[5]), fmaxf(wm[6], wm[7]));
            if (quarter == 0 && lane == 0) {
                as_global(t.absmax_m)[lb] = nam;
                as_global(t.absmax_v)[lb] = nav;
            }
            const BlockDiv dm(nam, kKeyScale, kKeyScaleInv), dv(nav, kKeyScale, kKeyScaleInv);
            const size_t e0 = (size_t)lb * kBlock;
            u32x2 mw, vw;
            if (dm.fast && dv.fast) requant8<true, true, MODE == ERI_ADAM8_MODE_BNB>(m, v, dm, dv, L, mw, vw);
            else requant8<false, true, MODE == ERI_ADAM8_MODE_BNB>(m, v, dm, dv, L, mw, vw);
            __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(t.m + e0 + o)));
            __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(t.v + e0 + o)));
        }
    }
}

namespace {

template <bool BF16, bool GBF16, int MODE, bool EXACT>
int launch_flags(bool wd, bool gs, const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                 const void *img, const float *dev_scale, uint32_t grid, uint32_t teams, hipStream_t s) {
#define ERI_GO(W, G)                                                                                                     \
    do {                                                                                                                 \
        hipLaunchKernelGGL((adam8_step_split_kernel<BF16, GBF16, MODE, EXACT, W, G>), dim3(grid), dim3(1024), 0, s, rows, n_rows, \
                           total_blocks, h, static_cast<const uint4 *>(img), dev_scale, teams);                           \
        return (int)hipGetLastError();                                                                                   \
    } while (0)
    if (wd) { if (gs) ERI_GO(true, true); ERI_GO(true, false); }
    if (gs) ERI_GO(false, true);
    ERI_GO(false, false);
#undef ERI_GO
}

} // namespace

int launch_step_split(int layout, int mode, bool exact, bool wd, bool gs, const DevTensor *rows, uint32_t n_rows,
                      uint32_t total_blocks, const EriAdam8Hyper &h, const void *img, const float *dev_scale, uint32_t grid,
                      uint32_t teams, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
#define ERI_ARGS wd, gs, rows, n_rows, total_blocks, h, img, dev_scale, grid, teams, s
    if (layout == kLayoutF32) { // fp32 parameters always take the IEEE square root and division
        if (mode == ERI_ADAM8_MODE_BNB) return launch_flags<false, false, ERI_ADAM8_MODE_BNB, true>(ERI_ARGS);
        if (mode == ERI_ADAM8_MODE_L2) return launch_flags<false, false, ERI_ADAM8_MODE_L2, true>(ERI_ARGS);
        return launch_flags<false, false, ERI_ADAM8_MODE_ERI, true>(ERI_ARGS);
    }
    // mode L2 always takes the IEEE chain
#define ERI_BF16(G)                                                                                                          \
    do {                                                                                                                     \
        if (mode == ERI_ADAM8_MODE_BNB)                                                                                      \
            return exact ? launch_flags<true, G, ERI_ADAM8_MODE_BNB, true>(ERI_ARGS) : launch_flags<true, G, ERI_ADAM8_MODE_BNB, false>(ERI_ARGS); \
        if (mode == ERI_ADAM8_MODE_L2) return launch_flags<true, G, ERI_ADAM8_MODE_L2, true>(ERI_ARGS);                        \
        return exact ? launch_flags<true, G, ERI_ADAM8_MODE_ERI, true>(ERI_ARGS) : launch_flags<true, G, ERI_ADAM8_MODE_ERI, false>(ERI_ARGS); \
    } while (0)
    if (layout == kLayoutBF16) ERI_BF16(true);
    ERI_BF16(false);
#undef ERI_BF16
#undef ERI_ARGS
}

} // namespace eri
