/* The software-pipelined step kernel: the benchmark kernel.  Compiled three times, once per layout of the
 * rows (-DERI_PIPE_LAYOUT=1: bf16 parameters and gradients, 2: bf16 parameters with fp32 gradients, 0: fp32
 * parameters and gradients), so that the three build in parallel. */
#include "eri_adam8_inline.h"

#if !defined(ERI_PIPE_LAYOUT) || ERI_PIPE_LAYOUT < 0 || ERI_PIPE_LAYOUT > 2
#error "compile with -DERI_PIPE_LAYOUT=0, 1 or 2"
#endif

namespace eri {

static_assert(kLayoutF32 == 0 && kLayoutBF16 == 1 && kLayoutBF16GradF32 == 2, "ERI_PIPE_LAYOUT names a Layout");
constexpr bool kParamBf16 = ERI_PIPE_LAYOUT != kLayoutF32;
constexpr bool kGradBf16 = ERI_PIPE_LAYOUT == kLayoutBF16;

// ------------------------------------------------------------------------------------------
// software-pipelined step kernel for bf16 tensors
//
// Same arithmetic as adam8_step_kernel, but a wave issues the loads of its NEXT block after the
// update half of the current block (when the raw words of the current block are dead) and before
// the requantisation half, so it always has 48 bytes per lane in flight while it computes.  The
// registers of the raw words are the ones just freed, so the pipeline costs no copies; it needs
// 48 (raw) + 64 (moments) + temporaries at its peak, hence three waves per SIMD (768 threads).
// With fp32 gradients the raw words of a block are 64 registers, with fp32 parameters too 80, which no
// longer fits beside the moments in the 170 registers of three waves per SIMD: those instantiations run
// two waves per SIMD (512 threads), each with 24 or 20 KB of its next block in flight.
// ------------------------------------------------------------------------------------------

constexpr uint32_t kPipeThreads = kGradBf16 ? 768 : 512;
#if ERI_PIPE_LAYOUT == 1
#define ERI_PIPE_KERNEL adam8_step_pipelined_kernel
#elif ERI_PIPE_LAYOUT == 2
#define ERI_PIPE_KERNEL adam8_step_pipelined_grad_f32_kernel
#else
#define ERI_PIPE_KERNEL adam8_step_pipelined_f32_kernel
#endif

/* One lane's eight shadow values of one quarter block: shadow = d*shadow + (1-d)*p', each operation rounded
 * on its own, the result rounded to bf16. */
__device__ __forceinline__ void ema_quarter(void *shadow, size_t e0, int c, uint32_t lane, const u32x4 &old, const u32x4 &pnew,
                                            float decay) {
    const float omd = 1.0f - decay; // ema_enhanced.rs:96
    Raw8<true> so, pn;
    so.w = old;
    pn.w = pnew;
    float sv[8], pv[8], out[8];
    so.unpack(sv);
    pn.unpack(pv);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        float a = sv[k] * decay;
        float b = pv[k] * omd;
        out[k] = a + b;
    }
    store8<true>(static_cast<char *>(shadow) + e0 * 2, c * 512 + lane * 8, out);
}

struct RawBlock {
    u32x4 p[kParamBf16 ? 4 : 8]; // bf16: one word per quarter block; fp32: two (elements 8*lane .. +3 and +4 .. +7)
    u32x4 g[kGradBf16 ? 4 : 8];
    u32x2 m[4], v[4];
    float a_m, a_v;
    /* Requests quarter c of block lb; the block's two absmax words ride with quarter 0. */
    __device__ __forceinline__ void issue_quarter(const DevTensor &t, uint32_t lb, int c, uint32_t lane) {
        const size_t e0 = (size_t)lb * kBlock;
        ERI_GLOBAL const u32x4 *pp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const char *>(t.p_in) + e0 * (kParamBf16 ? 2 : 4)));
        ERI_GLOBAL const u32x4 *gp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const char *>(t.g) + e0 * (kGradBf16 ? 2 : 4)));
        ERI_GLOBAL const u32x2 *mp = as_global(reinterpret_cast<const u32x2 *>(t.m + e0));
        ERI_GLOBAL const u32x2 *vp = as_global(reinterpret_cast<const u32x2 *>(t.v + e0));
        if (kParamBf16) {
            p[c] = __builtin_nontemporal_load(&pp[c * 64 + lane]); // each byte is touched once per step
        } else {
            p[2 * c] = pp[c * 128 + 2 * lane];
            p[2 * c + 1] = pp[c * 128 + 2 * lane + 1];
        }
        if (kGradBf16) {
            g[c] = __builtin_nontemporal_load(&gp[c * 64 + lane]);
        } else {
            // a lane's two words share cache lines with its neighbours' across the two instructions, so
            // these stay ordinary loads: streamed, the second instruction would fetch every line again
            g[2 * c] = gp[c * 128 + 2 * lane];
            g[2 * c + 1] = gp[c * 128 + 2 * lane + 1];
        }
        m[c] = __builtin_nontemporal_load(&mp[c * 64 + lane]);
        v[c] = __builtin_nontemporal_load(&vp[c * 64 + lane]);
        if (c == 0) {
            a_m = as_global(t.absmax_m)[lb];
            a_v = as_global(t.absmax_v)[lb];
        }
    }
    __device__ __forceinline__ void issue(const DevTensor &t, uint32_t lb, uint32_t lane) {
#pragma unroll
        for (int c = 0; c < 4; ++c) issue_quarter(t, lb, c, lane);
    }
};

/* EMA: rows that carry a shadow also get shadow = d*shadow + (1-d)*p' (src/trainers/ema_enhanced.rs:91-100),
 * p' being the parameter as it is stored (rounded to bf16). */
template <int MODE, bool EXACT, bool WD, bool GS, bool EMA>
__global__ __launch_bounds__(kPipeThreads) void ERI_PIPE_KERNEL(const DevTensor *__restrict__ rows,
                                                                   uint32_t n_rows, uint32_t total_blocks,
                                                                   EriAdam8Hyper h_in,
                                                                   const uint4 *__restrict__ lds_image,
                                                                   const float *__restrict__ dev_scale,
                                                                   uint32_t chunks) {
    ERI_LDS_IMAGE;
    const StepHyper h = make_step_hyper<MODE>(h_in);
    // Where the next block's loads go out.  The instantiations of the reference's own update request each quarter
    // of the next block as soon as the same quarter of this one has been consumed (its registers are free from
    // then on), so every load has a whole block's time to arrive; measured 1-4 % faster on 2.6 B parameters,
    // 1 % with fp32 gradients, 1.2-1.6 % with fp32 parameters, 0.6-0.9 % with the exact chain, neutral on 12 B
    // bf16 parameters with default flags.  With the EMA or another mode inside the loop that order costs
    // registers (12-80 bytes of scratch per lane) and time: those request the whole block after the update half.
    constexpr bool kEarly = MODE == ERI_ADAM8_MODE_ERI && !EMA;
    // Per wave, the 2 x 256 values a state code of the block at hand can stand for, already multiplied by the
    // block's absmax and by beta: (MAP[c] * absmax) * beta, the first two operations of both moment
    // updates, done once per code (8 per lane) instead of once per element (64 per lane).
    __shared__ float decayed[12][2][256];
    // clip factor left on the device by the gradient-norm pass (1.0 when there is none)
    const float tscale = (GS && dev_scale) ? *dev_scale : 1.0f;
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

    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t stride = gridDim.x * waves_per_wg;
    const BlockDiv dbc1(h.bc1), dbc2(h.bc2);
    float(*const mine)[256] = decayed[threadIdx.x / kWave];
    const f32x4 base_s = reinterpret_cast<const f32x4 *>(L.map_s)[lane]; // codes 4*lane .. 4*lane + 3
    const f32x4 base_u = reinterpret_cast<const f32x4 *>(L.map_u)[lane];

    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    // partial last blocks first: one per row at most, handed out from the last wave backwards -- the
    // waves at the end of each range are the ones that get one full block fewer when the blocks do not
    // divide evenly, so the slower element-wise tail lands where there is slack
    for (uint32_t r = stride - 1 - wave; r < n_rows; r += stride) {
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        if (n != 0) {
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            tail_block<kParamBf16, MODE, EXACT, WD, GS, true, kGradBf16>(t, (uint32_t)(t.numel / kBlock), n, lane, h, gscale, dbc1, dbc2, L);
            if (EMA && t.shadow != nullptr) { // the partial block's shadow, element by element, from the parameters just stored
                const size_t e0 = (size_t)(t.numel / kBlock) * kBlock;
                const float omd = 1.0f - h.ema_decay;
                for (uint32_t i = lane; i < n; i += kWave) {
                    const float a = load1<true>(t.shadow, e0 + i) * h.ema_decay;
                    const float b = load1<true>(t.p, e0 + i) * omd;
                    as_global(static_cast<uint16_t *>(t.shadow))[e0 + i] = (uint16_t)bf16_bits(a + b);
                }
            }
        }
    }
    const BlockWalk walk(total_blocks, chunks);
    uint32_t blk = walk.first;
    if (blk >= walk.end) return;

    uint32_t ti = 0, t_end = 0;
    DevTensor t;
    const BlockRowMap map(rows, n_rows);
    map.seek(rows, blk, ti, t, t_end);
    uint32_t nti = ti, nt_end = t_end;
    DevTensor nt = t;
    RawBlock raw;
    raw.issue(t, blk - t.full_start, lane);
    while (true) {
        // the block after this one; past the end the wave re-reads its last block (the loads must
        // stay unconditional so that the raw registers have a single definition in the loop)
        const uint32_t nblk = blk + walk.stride;
        const bool more = nblk < walk.end;
        const uint32_t pblk = more ? nblk : blk;
        map.seek(rows, pblk, nti, nt, nt_end);

        const uint32_t lb = blk - t.full_start;
        const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
        const size_t e0 = (size_t)lb * kBlock;
        char *p = static_cast<char *>(t.p) + e0 * (kParamBf16 ? 2 : 4);
        uint8_t *mc = t.m + e0;
        uint8_t *vc = t.v + e0;
        float mf[32], vf[32];
        u32x4 pw[4]; // updated parameters, packed, stored after the next block's loads are out
        float lm = 0.0f, lv = 0.0f;
        const float a_m = raw.a_m, a_v = raw.a_v;
        {
            f32x4 ds, du;
            ds.x = (base_s.x * a_m) * h.beta1; ds.y = (base_s.y * a_m) * h.beta1;
            ds.z = (base_s.z * a_m) * h.beta1; ds.w = (base_s.w * a_m) * h.beta1;
            du.x = (base_u.x * a_v) * h.beta2; du.y = (base_u.y * a_v) * h.beta2;
            du.z = (base_u.z * a_v) * h.beta2; du.w = (base_u.w * a_v) * h.beta2;
            reinterpret_cast<f32x4 *>(mine[0])[lane] = ds;
            reinterpret_cast<f32x4 *>(mine[1])[lane] = du;
        }
        // EMA: the shadow's words are requested first and used quarter by quarter in the update half, where the
        // registers of the moments are still filling up (in the requantisation half, beside the next block's
        // words, they did not fit: 104-152 bytes of scratch per lane)
        u32x4 sh[4];
        const bool with_shadow = EMA && t.shadow != nullptr;
        if (EMA && with_shadow) {
            ERI_GLOBAL const u32x4 *sp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(t.shadow) + e0));
#pragma unroll
            for (int c = 0; c < 4; ++c) sh[c] = __builtin_nontemporal_load(&sp[c * 64 + lane]);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float pv[8], gv[8], pn[8];
            if (kParamBf16) {
                Raw8<true> pr;
                pr.w = raw.p[c];
                pr.unpack(pv);
            } else {
                const u32x4 pa = raw.p[kParamBf16 ? c : 2 * c], pb = raw.p[kParamBf16 ? c : 2 * c + 1];
                pv[0] = u2f(pa.x); pv[1] = u2f(pa.y); pv[2] = u2f(pa.z); pv[3] = u2f(pa.w);
                pv[4] = u2f(pb.x); pv[5] = u2f(pb.y); pv[6] = u2f(pb.z); pv[7] = u2f(pb.w);
            }
            if (kGradBf16) {
                Raw8<true> gr;
                gr.w = raw.g[c];
                gr.unpack(gv);
            } else {
                const u32x4 ga = raw.g[kGradBf16 ? c : 2 * c], gb = raw.g[kGradBf16 ? c : 2 * c + 1];
                gv[0] = u2f(ga.x); gv[1] = u2f(ga.y); gv[2] = u2f(ga.z); gv[3] = u2f(ga.w);
                gv[4] = u2f(gb.x); gv[5] = u2f(gb.y); gv[6] = u2f(gb.z); gv[7] = u2f(gb.w);
            }
            // one flag per element: flagged elements are put right quarter by quarter (before the shadow uses
            // them), and the exact chain runs for the flagged positions only
            Redo8 redo;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float t1 = lds_float_at(mine[0], code_offset(raw.m[c], k));
                const float t3 = lds_float_at(mine[1], code_offset(raw.v[c], k));
                float m, v;
                uint64_t flagged = 0;
                adam_elem_decayed<MODE, EXACT, kParamBf16, WD, GS>(pv[k], gv[k], t1, t3, h, gscale, dbc1, dbc2, m, v, pn[k], flagged);
                redo.set(k, flagged);
                mf[c * 8 + k] = m;
                vf[c * 8 + k] = v;
                lm = fmaxf(lm, __builtin_fabsf(m));
                lv = fmaxf(lv, __builtin_fabsf(v));
            }
            if (kParamBf16 && MODE == ERI_ADAM8_MODE_L2 && h.l2_all_exact) redo.set_all();
            if (kParamBf16 && redo.any) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (redo.lanes[k] && redo.mine(k))
                        pn[k] = param_exact<MODE, WD, true>(pv[k], mf[c * 8 + k], vf[c * 8 + k], h, dbc1, dbc2);
            }
            if (kParamBf16) {
                pw[c].x = bf16_pair(pn[0], pn[1]);
                pw[c].y = bf16_pair(pn[2], pn[3]);
                pw[c].z = bf16_pair(pn[4], pn[5]);
                pw[c].w = bf16_pair(pn[6], pn[7]);
            } else { // fp32 parameters are final here (they take the exact chain): stored quarter by quarter
                store8<false>(p, c * 512 + lane * 8, pn);
            }
            if (EMA && with_shadow) ema_quarter(t.shadow, e0, c, lane, sh[c], pw[c], h.ema_decay);
            if (kEarly) { // the quarter's raw words are dead: the next block's quarter takes their registers now
                raw.issue_quarter(nt, pblk - nt.full_start, c, lane);
                if (kParamBf16) __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
            }
        }
        float nam = lm, nav = lv;
        wave_max2(nam, nav);
        if (lane == 0) {
            as_global(t.absmax_m)[lb] = nam;
            as_global(t.absmax_v)[lb] = nav;
        }
        if (!kEarly) raw.issue(nt, pblk - nt.full_start, lane); // prefetch: in flight during the requantisation
        if (kParamBf16 && !kEarly) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
        }
        const BlockDiv dm(nam, kKeyScale, kKeyScaleInv), dv(nav, kKeyScale, kKeyScaleInv);
        if (dm.fast && dv.fast) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t o = c * 512 + lane * 8;
                u32x2 mw, vw;
                requant8<true, true, MODE == ERI_ADAM8_MODE_BNB>(mf + c * 8, vf + c * 8, dm, dv, L, mw, vw);
                __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(mc + o)));
                __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(vc + o)));
            }
        } else {
            for (int c = 0; c < 4; ++c) {
                const uint32_t o = c * 512 + lane * 8;
                u32x2 mw, vw;
                requant8<false, true, MODE == ERI_ADAM8_MODE_BNB>(mf + c * 8, vf + c * 8, dm, dv, L, mw, vw);
                __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(mc + o)));
                __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(vc + o)));
            }
        }
        if (!more) break;
        blk = nblk;
        t = nt;
    }
}

namespace {

template <int MODE, bool EXACT, bool WD, bool GS, bool EMA = false>
int launch_pipelined(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                     const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    if (wg > kPipeThreads) wg = kPipeThreads;
    hipLaunchKernelGGL((ERI_PIPE_KERNEL<MODE, EXACT, WD, GS, EMA>), dim3(grid), dim3(wg), 0, s, rows, n_rows, total_blocks, h,
                       static_cast<const uint4 *>(lds_image), dev_scale, chunks_for(grid));
    return (int)hipGetLastError();
}

template <int MODE, bool EXACT>
int launch_flags(bool wd, bool gs, bool ema, const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                 const void *img, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    if constexpr (MODE == ERI_ADAM8_MODE_ERI && kParamBf16) { // the EMA is built into the reference's own update, on bf16 parameters
        if (ema) {
            if (wd) {
                if (gs) return launch_pipelined<MODE, EXACT, true, true, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
                return launch_pipelined<MODE, EXACT, true, false, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
            }
            if (gs) return launch_pipelined<MODE, EXACT, false, true, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
            return launch_pipelined<MODE, EXACT, false, false, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
        }
    }
    if (wd) {
        if (gs) return launch_pipelined<MODE, EXACT, true, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
        return launch_pipelined<MODE, EXACT, true, false>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
    }
    if (gs) return launch_pipelined<MODE, EXACT, false, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
    return launch_pipelined<MODE, EXACT, false, false>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
}

} // namespace

/* All three modes.  (The coupled-decay mode fits the register budget since its bias corrections became
 * products in the fast chain: 168 registers, no scratch; with the two divisions it spilled 80-232 B per lane.) */
#if ERI_PIPE_LAYOUT == 1
int launch_step_pipelined(int mode, bool exact, bool wd, bool gs, bool ema, const DevTensor *rows, uint32_t n_rows,
                          uint32_t total_blocks, const EriAdam8Hyper &h, const void *img, const float *dev_scale,
                          uint32_t grid, uint32_t wg, void *stream) {
#elif ERI_PIPE_LAYOUT == 2
int launch_step_pipelined_grad_f32(int mode, bool exact, bool wd, bool gs, bool ema, const DevTensor *rows, uint32_t n_rows,
                                   uint32_t total_blocks, const EriAdam8Hyper &h, const void *img,
                                   const float *dev_scale, uint32_t grid, uint32_t wg, void *stream) {
#else
int launch_step_pipelined_f32(int mode, bool wd, bool gs, const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks,
                              const EriAdam8Hyper &h, const void *img, const float *dev_scale, uint32_t grid,
                              uint32_t wg, void *stream) {
    const bool ema = false;   // fp32 rows get their EMA from the sweep
    constexpr bool exact = true; // fp32 parameters always take the IEEE square root and division
#endif
    hipStream_t s = static_cast<hipStream_t>(stream);
#define ERI_ARGS wd, gs, ema, rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s
#if ERI_PIPE_LAYOUT == 0
    if (mode == ERI_ADAM8_MODE_L2) return launch_flags<ERI_ADAM8_MODE_L2, exact>(ERI_ARGS);
    if (mode == ERI_ADAM8_MODE_BNB) return launch_flags<ERI_ADAM8_MODE_BNB, exact>(ERI_ARGS);
    return launch_flags<ERI_ADAM8_MODE_ERI, exact>(ERI_ARGS);
#else
    if (mode == ERI_ADAM8_MODE_L2) return launch_flags<ERI_ADAM8_MODE_L2, true>(ERI_ARGS); // its fast chain always checks itself
    if (mode == ERI_ADAM8_MODE_BNB)
        return exact ? launch_flags<ERI_ADAM8_MODE_BNB, true>(ERI_ARGS) : launch_flags<ERI_ADAM8_MODE_BNB, false>(ERI_ARGS);
    return exact ? launch_flags<ERI_ADAM8_MODE_ERI, true>(ERI_ARGS) : launch_flags<ERI_ADAM8_MODE_ERI, false>(ERI_ARGS);
#endif
#undef ERI_ARGS
}

} // namespace eri
