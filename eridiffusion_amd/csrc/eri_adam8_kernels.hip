/*
 * Dispatch of the step to its two kernels, and the smaller kernels around it: state creation,
 * checkpoint quantisation, the gradient-norm pass, the quantisation-error pass, the 32-bit step and the
 * EMA sweep.
 */
#include "eri_adam8_inline.h"

namespace eri {

/* The one case in which the EMA runs inside the step kernel: the prefetching kernel in mode ERI, on bf16
 * parameters (with bf16 or fp32 gradients). */
bool step_fuses_ema(uint32_t total_blocks, int layout, const EriAdam8Hyper &h, uint32_t compute_units) {
    if ((h.flags & ERI_ADAM8_FLAG_EMA) == 0 || !layout_param_bf16(layout) || h.mode != ERI_ADAM8_MODE_ERI) return false;
    if (h.flags & (ERI_ADAM8_FLAG_BSEARCH | ERI_ADAM8_FLAG_NO_PIPELINE)) return false;
    const bool few = (uint64_t)total_blocks <= (uint64_t)compute_units * (uint64_t)kSplitBlocksPerCu;
    return (h.flags & ERI_ADAM8_FLAG_ONE_WAVE) != 0 || !few;
}

/* Whether a bf16 table that qualifies for the prefetching kernel is large enough to gain from it.  A step
 * that carries the EMA stays on the prefetching kernel at every size: it is the one that fuses it. */
static bool prefetch_pays(uint32_t total_blocks, const EriAdam8Hyper &h, uint32_t compute_units) {
    if (h.flags & (ERI_ADAM8_FLAG_ONE_WAVE | ERI_ADAM8_FLAG_EMA)) return true;
    return (uint64_t)total_blocks > (uint64_t)compute_units * (uint64_t)kPrefetchBlocksPerCu;
}

int launch_step(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int layout,
                const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg,
                uint32_t compute_units, void *stream) {
    const bool bf16 = layout_param_bf16(layout);
    const bool mixed = layout == kLayoutBF16GradF32; // F32 gradients for BF16 parameters
    const bool gs = (h.flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
    // Four waves share each block where one wave per block would leave the chip idle: tables of few blocks.
    // The flags that name a kernel (cross-checks) keep their meaning; bf16 parameters with fp32 gradients
    // have no binary-search variant of the one-wave kernel and stay on this one for those flags.
    const bool one_wave = (h.flags & ERI_ADAM8_FLAG_ONE_WAVE) != 0;
    const bool kernel_named = (h.flags & (ERI_ADAM8_FLAG_BSEARCH | ERI_ADAM8_FLAG_NO_PIPELINE)) != 0;
    const bool few = (uint64_t)total_blocks <= (uint64_t)compute_units * (uint64_t)kSplitBlocksPerCu;
    if ((mixed && (h.flags & ERI_ADAM8_FLAG_BSEARCH) != 0) || (!kernel_named && !one_wave && few)) {
        const bool bnb = h.mode == ERI_ADAM8_MODE_BNB;
        const bool wd_s = bnb ? h.weight_decay != 1.0f : h.weight_decay > 0.0f;
        const bool exact_s = !bf16 || (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0;
        // Up to four blocks per workgroup at a time (a team of four waves each), but no more than it takes to
        // give every compute unit a workgroup: 512 blocks on 256 units run as 256 workgroups of two teams.
        uint32_t teams = (total_blocks + compute_units - 1) / compute_units;
        teams = teams < 1 ? 1 : teams > 4 ? 4 : teams;
        uint32_t need = (total_blocks + teams - 1) / teams;
        const uint32_t for_tails = (n_rows + 15) / 16;
        if (need < for_tails) need = for_tails;
        if (need > compute_units) need = compute_units;
        if (need == 0) need = 1;
        return launch_step_split(layout, h.mode, exact_s, wd_s, gs, rows, n_rows, total_blocks, h, lds_image, dev_scale, need,
                                 teams, stream);
    }
    if (mixed) {
        const bool wd_m = h.mode == ERI_ADAM8_MODE_BNB ? h.weight_decay != 1.0f : h.weight_decay > 0.0f;
        if ((h.flags & ERI_ADAM8_FLAG_NO_PIPELINE) == 0 && prefetch_pays(total_blocks, h, compute_units))
            return launch_step_pipelined_grad_f32(h.mode, (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0, wd_m, gs,
                                                  step_fuses_ema(total_blocks, layout, h, compute_units), rows, n_rows,
                                                  total_blocks, h, lds_image, dev_scale, grid, wg, stream);
        return launch_step_plain_bf16(h.mode, (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0, wd_m, gs, true, true, rows, n_rows,
                                      total_blocks, h, lds_image, dev_scale, grid, wg, stream);
    }
    if (h.mode == ERI_ADAM8_MODE_BNB) { // slot table only; the decay is a factor
        const bool wd = h.weight_decay != 1.0f;
        const bool exact = (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0;
        if (bf16 && !kernel_named && prefetch_pays(total_blocks, h, compute_units))
            return launch_step_pipelined(h.mode, exact, wd, gs, false, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
        if (bf16) return launch_step_plain_bf16(h.mode, exact, wd, gs, true, false, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
        if (!kernel_named && prefetch_pays(total_blocks, h, compute_units))
            return launch_step_pipelined_f32(h.mode, wd, gs, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
        return launch_step_plain_f32(h.mode, wd, gs, true, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
    }
    const bool wd = h.weight_decay > 0.0f;
    const bool exact = (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0;
    const bool keytab = (h.flags & ERI_ADAM8_FLAG_BSEARCH) == 0;
    if (!bf16 && !kernel_named && prefetch_pays(total_blocks, h, compute_units))
        return launch_step_pipelined_f32(h.mode, wd, gs, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
    if (!bf16) return launch_step_plain_f32(h.mode, wd, gs, keytab, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
    if (keytab && (h.flags & ERI_ADAM8_FLAG_NO_PIPELINE) == 0 && prefetch_pays(total_blocks, h, compute_units))
        return launch_step_pipelined(h.mode, exact, wd, gs, step_fuses_ema(total_blocks, layout, h, compute_units), rows, n_rows,
                                     total_blocks, h, lds_image, dev_scale, grid, wg, stream);
    return launch_step_plain_bf16(h.mode, exact, wd, gs, keytab, false, rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, stream);
}

// ------------------------------------------------------------------------------------------
// state initialisation and blockwise (de)quantisation for checkpoint traffic
// ------------------------------------------------------------------------------------------

__global__ void state_init_kernel(uint8_t *m, uint8_t *v, float *am, float *av, uint64_t numel, uint64_t nblocks) {
    const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint64_t n = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = tid; i < numel; i += n) {
        m[i] = 127;
        v[i] = 0;
    }
    for (uint64_t b = tid; b < nblocks; b += n) {
        am[b] = 0.0f;
        av[b] = 0.0f;
    }
}

// ------------------------------------------------------------------------------------------
// diagnostics: the memory traffic of one step over bf16 rows and nothing else
// ------------------------------------------------------------------------------------------

/* Every full block of the table is read and written as the step kernel reads and writes it -- the launch shape
 * of the prefetching kernel (one workgroup of 768 threads per compute unit, one range of the block list per die),
 * 128-bit non-temporal loads of parameters and gradients, 64-bit ones of the two code arrays, the two absmax
 * words, all of a block's loads in flight before its first store -- with no arithmetic between load and store.
 * Parameters, codes and absmax are written back with the bits they had (`zero` is 0 at run time, which the
 * compiler cannot know, so neither the loads of the gradients nor the stores fall away).  What this launch takes
 * is what the memory system gives the step's mix of four read and three written streams in the placement at
 * hand; the step kernel cannot be faster than that. */
__global__ __launch_bounds__(768) void traffic_probe_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                            uint32_t total_blocks, uint32_t chunks, uint32_t zero) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const BlockWalk walk(total_blocks, chunks);
    const BlockRowMap map(rows, n_rows);
    uint32_t ti = 0, t_end = 0;
    DevTensor t;
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        map.seek(rows, blk, ti, t, t_end);
        const uint32_t lb = blk - t.full_start;
        const size_t e0 = (size_t)lb * kBlock;
        ERI_GLOBAL u32x4 *pp = as_global(reinterpret_cast<u32x4 *>(static_cast<char *>(t.p) + e0 * 2));
        ERI_GLOBAL const u32x4 *gp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const char *>(t.g) + e0 * 2));
        ERI_GLOBAL u32x2 *mp = as_global(reinterpret_cast<u32x2 *>(t.m + e0));
        ERI_GLOBAL u32x2 *vp = as_global(reinterpret_cast<u32x2 *>(t.v + e0));
        u32x4 p[4], g[4];
        u32x2 m[4], v[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            p[c] = __builtin_nontemporal_load(&pp[c * 64 + lane]);
            g[c] = __builtin_nontemporal_load(&gp[c * 64 + lane]);
            m[c] = __builtin_nontemporal_load(&mp[c * 64 + lane]);
            v[c] = __builtin_nontemporal_load(&vp[c * 64 + lane]);
        }
        const uint32_t a_m = f2u(as_global(t.absmax_m)[lb]), a_v = f2u(as_global(t.absmax_v)[lb]);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            __builtin_nontemporal_store(p[c] ^ (g[c] & zero), &pp[c * 64 + lane]);
            __builtin_nontemporal_store(m[c] ^ zero, &mp[c * 64 + lane]);
            __builtin_nontemporal_store(v[c] ^ zero, &vp[c * 64 + lane]);
        }
        if (lane == 0) {
            as_global(t.absmax_m)[lb] = u2f(a_m ^ zero);
            as_global(t.absmax_v)[lb] = u2f(a_v ^ zero);
        }
    }
}

int launch_traffic_probe(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, uint32_t grid, void *stream) {
    hipLaunchKernelGGL(traffic_probe_kernel, dim3(grid), dim3(768), 0, static_cast<hipStream_t>(stream), rows, n_rows,
                       total_blocks, chunks_for(grid), 0u);
    return (int)hipGetLastError();
}

__global__ void fill_zero_kernel(uint4 *p, uint64_t words) {
    const uint64_t n = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < words; i += n) p[i] = uint4{0u, 0u, 0u, 0u};
}

int launch_fill_zero(void *p, size_t bytes, void *stream) {
    if (bytes == 0) return 0;
    if ((((uintptr_t)p) | bytes) & 15u) return (int)hipErrorInvalidValue;
    const uint64_t words = bytes / 16;
    uint64_t grid = (words + 255) / 256;
    if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(fill_zero_kernel, dim3((uint32_t)grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<uint4 *>(p), words);
    return (int)hipGetLastError();
}

int launch_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel, void *stream) {
    const uint64_t nblocks = (numel + kBlock - 1) / kBlock;
    uint64_t grid = (numel + 255) / 256;
    if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(state_init_kernel, dim3((uint32_t)grid), dim3(256), 0, static_cast<hipStream_t>(stream), m,
                       v, absmax_m, absmax_v, numel, nblocks);
    return (int)hipGetLastError();
}

__global__ void dequantize_kernel(const uint8_t *codes, const float *absmax, uint64_t numel, float *out,
                                  const float *map) {
    __shared__ float lmap[256];
    lmap[threadIdx.x] = map[threadIdx.x];
    __syncthreads();
    const uint64_t n = (uint64_t)gridDim.x * blockDim.x;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < numel; i += n)
        out[i] = lmap[codes[i]] * absmax[i / kBlock];
}

int launch_dequantize(const uint8_t *codes, const float *absmax, int signed_map, uint64_t numel, float *out,
                      const void *lds_image, void *stream) {
    const float *map = reinterpret_cast<const float *>(static_cast<const char *>(lds_image) +
                                                       (signed_map ? kOffMapS : kOffMapU));
    uint64_t grid = (numel + 255) / 256;
    if (grid > 16384) grid = 16384;
    hipLaunchKernelGGL(dequantize_kernel, dim3((uint32_t)grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       codes, absmax, numel, out, map);
    return (int)hipGetLastError();
}

/* One wavefront per block: absmax by DPP, then the nearest code by binary search. */
__global__ void quantize_kernel(const float *x, uint64_t numel, uint64_t nblocks, uint8_t *codes, float *absmax,
                                const float *mid) {
    __shared__ float lmid[256];
    lmid[threadIdx.x] = mid[threadIdx.x];
    __syncthreads();
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint64_t wave = (uint64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    const uint64_t nw = (uint64_t)gridDim.x * (blockDim.x / kWave);
    for (uint64_t b = wave; b < nblocks; b += nw) {
        const uint64_t e0 = b * kBlock;
        const uint32_t n = (uint32_t)((numel - e0) < kBlock ? (numel - e0) : kBlock);
        float a = 0.0f;
        for (uint32_t i = lane; i < n; i += kWave) a = fmaxf(a, __builtin_fabsf(x[e0 + i]));
        a = wave_max(a);
        for (uint32_t i = lane; i < n; i += kWave) {
            const float q = a == 0.0f ? 0.0f : x[e0 + i] / a;
            codes[e0 + i] = (uint8_t)code_bsearch(q, lmid);
        }
        if (lane == 0) absmax[b] = a;
    }
}

int launch_quantize(const float *x, int signed_map, uint64_t numel, uint8_t *codes, float *absmax,
                    const void *lds_image, void *stream) {
    const float *mid = reinterpret_cast<const float *>(static_cast<const char *>(lds_image) +
                                                       (signed_map ? kOffMidS : kOffMidU));
    const uint64_t nblocks = (numel + kBlock - 1) / kBlock;
    uint64_t grid = (nblocks + 3) / 4;
    if (grid > 8192) grid = 8192;
    hipLaunchKernelGGL(quantize_kernel, dim3((uint32_t)grid), dim3(256), 0, static_cast<hipStream_t>(stream), x,
                       numel, nblocks, codes, absmax, mid);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// global gradient norm over the launch table (the trainers' clip_gradients,
// src/trainers/pipeline_flux_lora_sequential.rs:1198-1213,1939-1950), without a host round trip:
// pass 1 forms one fp32 sum of squares per block and adds a wave's blocks in f64, pass 2 adds the waves'
// partials and writes the norm and
// the clip factor to device memory, where the step kernel reads it.
// ------------------------------------------------------------------------------------------

/* 1.0 for NaN and +-infinity, else 0.0 */
__device__ __forceinline__ float not_finite(float x) { return (__builtin_fabsf(x) <= 3.4028234e38f) ? 0.0f : 1.0f; }

__device__ __forceinline__ float wave_sum(float x) {
    // fixed reduction tree, so the result does not depend on scheduling
    x += dpp_mov<0xB1, 0xf>(x);
    x += dpp_mov<0x4E, 0xf>(x);
    x += dpp_mov<0x141, 0xf>(x);
    x += dpp_mov<0x140, 0xf>(x); // every lane: its row's sum
    float r = u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(x), 15));
    r += u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(x), 31));
    r += u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(x), 47));
    r += u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(x), 63));
    return r;
}

template <bool BF16>
__global__ __launch_bounds__(1024) void grad_sumsq_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                         uint32_t total_blocks, double *__restrict__ partial,
                                                         uint32_t chunks) {
    // persistent: every wave adds the fp32 sums of its blocks in f64 and leaves one partial
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    const uint32_t stride = gridDim.x * waves_per_wg;
    double total = 0.0, bad = 0.0;
    for (uint32_t r = wave; r < n_rows; r += stride) { // partial last blocks
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        const size_t e0 = (size_t)(t.numel / kBlock) * kBlock;
        float acc = 0.0f, nf = 0.0f;
        for (uint32_t i = lane; i < n; i += kWave) {
            const float g = load1<BF16>(t.g, e0 + i);
            acc += g * g;
            nf += not_finite(g);
        }
        total += (double)wave_sum(acc);
        bad += (double)wave_sum(nf);
    }
    // full blocks, one load ahead: the next block's four words are in flight while this one is reduced
    const BlockWalk walk(total_blocks, chunks);
    if (walk.first < walk.end) {
        uint32_t ti = 0, t_end = 0;
        DevTensor t;
        Raw8<BF16> raw[4];
        const BlockRowMap map(rows, n_rows);
        {
            map.seek(rows, walk.first, ti, t, t_end);
            const size_t e0 = (size_t)(walk.first - t.full_start) * kBlock;
#pragma unroll
            for (int c = 0; c < 4; ++c) raw[c].load(static_cast<const char *>(t.g) + e0 * (BF16 ? 2 : 4), c * 512 + lane * 8);
        }
        for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
            Raw8<BF16> cur[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) cur[c] = raw[c];
            const uint32_t nblk = blk + walk.stride;
            if (nblk < walk.end) {
                map.seek(rows, nblk, ti, t, t_end);
                const size_t e0 = (size_t)(nblk - t.full_start) * kBlock;
#pragma unroll
                for (int c = 0; c < 4; ++c) raw[c].load(static_cast<const char *>(t.g) + e0 * (BF16 ? 2 : 4), c * 512 + lane * 8);
            }
            float acc = 0.0f;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float g[8];
                cur[c].unpack(g);
#pragma unroll
                for (int k = 0; k < 8; ++k) acc += g[k] * g[k];
            }
            const float block_sum = wave_sum(acc);
            total += (double)block_sum;
            if (not_finite(block_sum) != 0.0f) { // rare: count the NaN / infinite elements of this block
                float nf = 0.0f;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float g[8];
                    cur[c].unpack(g);
#pragma unroll
                    for (int k = 0; k < 8; ++k) nf += not_finite(g[k]);
                }
                bad += (double)wave_sum(nf);
            }
        }
    }
    if (lane == 0) {
        partial[2 * wave] = total;
        partial[2 * wave + 1] = bad;
    }
}

__global__ __launch_bounds__(1024) void grad_norm_finish_kernel(const double *__restrict__ partial, uint32_t n,
                                                                float max_norm, float denom_eps,
                                                                float *__restrict__ out /* norm, scale, u64 count */) {
    // partial holds, per wave of the first pass, the sum of squares and the count of non-finite elements
    __shared__ double sh[1024], shb[1024];
    double acc = 0.0, bad = 0.0;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        acc += partial[2 * i];
        bad += partial[2 * i + 1];
    }
    sh[threadIdx.x] = acc;
    shb[threadIdx.x] = bad;
    __syncthreads();
    for (uint32_t s = blockDim.x / 2; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            sh[threadIdx.x] += sh[threadIdx.x + s];
            shb[threadIdx.x] += shb[threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        const float norm = (float)sqrt(sh[0]);
        float scale = 1.0f;
        // clip only a finite norm above the limit (crates/training/src/optimizer.rs:79-84)
        if (max_norm > 0.0f && norm > max_norm && norm <= 3.4028234e38f) scale = max_norm / (norm + denom_eps);
        out[0] = norm;
        out[1] = scale;
        *reinterpret_cast<unsigned long long *>(out + 2) = (unsigned long long)shb[0];
    }
}

int launch_grad_sumsq(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, bool grad_bf16, double *partial,
                      uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (!grad_bf16)
        hipLaunchKernelGGL(grad_sumsq_kernel<false>, dim3(grid), dim3(kNormWaves * kWave), 0, s, rows, n_rows, total_blocks, partial, chunks_for(grid));
    else
        hipLaunchKernelGGL(grad_sumsq_kernel<true>, dim3(grid), dim3(kNormWaves * kWave), 0, s, rows, n_rows, total_blocks, partial, chunks_for(grid));
    return (int)hipGetLastError();
}

int launch_grad_norm_finish(const double *partial, uint32_t n, float max_norm, float denom_eps, float *out,
                            void *stream) {
    hipLaunchKernelGGL(grad_norm_finish_kernel, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream), partial, n,
                       max_norm, denom_eps, out);
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// quantisation error of the step that is about to run (quantization_stats,
// src/trainers/adam8bit_enhanced.rs:93-100,318-327): a read-only pass that forms the new moments
// exactly as the step will, quantises them, and adds |value - dequantised value| per row in f64.
// Diagnostics, not tuned: element by element, binary search.
// ------------------------------------------------------------------------------------------

__device__ __forceinline__ double wave_sum_f64(double x) {
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

template <bool BF16, int MODE, bool WD, bool GS>
__global__ __launch_bounds__(256) void quant_error_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                          uint32_t total_blocks, EriAdam8Hyper h_in,
                                                          const float *__restrict__ lds_image,
                                                          const float *__restrict__ dev_scale,
                                                          double *__restrict__ err /* [2 * n_rows] */, bool grad_f32) {
    const StepHyper h = make_step_hyper<MODE>(h_in);
    __shared__ float tab[1024]; // signed map, unsigned map, signed midpoints, unsigned midpoints
    for (uint32_t i = threadIdx.x; i < 1024; i += blockDim.x) tab[i] = lds_image[i];
    __syncthreads();
    const float *map_s = tab, *map_u = tab + 256, *mid_s = tab + 512, *mid_u = tab + 768;
    const float tscale = (GS && dev_scale) ? *dev_scale : 1.0f;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    const uint32_t stride = gridDim.x * waves_per_wg;
    const BlockDiv dbc1(h.bc1), dbc2(h.bc2);
    // every block of every row, partial ones included: rows are walked block by block
    uint32_t ti = 0;
    const uint32_t all_blocks = total_blocks + n_rows; // full blocks, then one (possibly empty) tail per row
    for (uint32_t w = wave; w < all_blocks; w += stride) {
        uint32_t lb, n;
        if (w < total_blocks) {
            ti = find_row(rows, n_rows, ti, w);
            lb = w - rows[ti].full_start;
            n = kBlock;
        } else {
            ti = w - total_blocks;
            lb = (uint32_t)(rows[ti].numel / kBlock);
            n = (uint32_t)(rows[ti].numel % kBlock);
            if (n == 0) continue;
        }
        const DevTensor t = rows[ti];
        const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
        const size_t e0 = (size_t)lb * kBlock;
        ERI_GLOBAL const uint8_t *mc = as_global(static_cast<const uint8_t *>(t.m));
        ERI_GLOBAL const uint8_t *vc = as_global(static_cast<const uint8_t *>(t.v));
        const float a_m = as_global(t.absmax_m)[lb];
        const float a_v = as_global(t.absmax_v)[lb];
        float lm = 0.0f, lv = 0.0f;
        for (uint32_t i = lane; i < n; i += kWave) {
            const size_t e = e0 + i;
            float m, v, pn;
            uint64_t unused = 0; // the exact chain never sets it
            const float gr = (BF16 && !grad_f32) ? load1<true>(t.g, e) : load1<false>(t.g, e);
            adam_elem<MODE, true, BF16, WD, GS>(load1<BF16>(t.p_in, e), gr, map_s[mc[e]] * a_m,
                                                map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn, unused);
            lm = fmaxf(lm, __builtin_fabsf(m));
            lv = fmaxf(lv, __builtin_fabsf(v));
        }
        float nam = lm, nav = lv;
        wave_max2(nam, nav);
        const BlockDiv dm(nam), dv(nav);
        double em = 0.0, ev = 0.0;
        for (uint32_t i = lane; i < n; i += kWave) {
            const size_t e = e0 + i;
            float m, v, pn;
            uint64_t unused = 0; // the exact chain never sets it
            const float gr = (BF16 && !grad_f32) ? load1<true>(t.g, e) : load1<false>(t.g, e);
            adam_elem<MODE, true, BF16, WD, GS>(load1<BF16>(t.p_in, e), gr, map_s[mc[e]] * a_m,
                                                map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn, unused);
            const float qm = map_s[code_bsearch(dm.div_slow(m), mid_s)] * nam;
            const float qv = map_u[code_bsearch(dv.div_slow(v), mid_u)] * nav;
            em += (double)__builtin_fabsf(m - qm);
            ev += (double)__builtin_fabsf(v - qv);
        }
        em = wave_sum_f64(em);
        ev = wave_sum_f64(ev);
        if (lane == 0) {
            atomicAdd(&err[2 * ti], em);
            atomicAdd(&err[2 * ti + 1], ev);
        }
    }
}

__global__ void zero_f64_kernel(double *x, uint32_t n) {
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) x[i] = 0.0;
}

int launch_quant_error(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int layout,
                       const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, double *err,
                       uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float *img = static_cast<const float *>(lds_image);
    hipLaunchKernelGGL(zero_f64_kernel, dim3(64), dim3(256), 0, s, err, 2 * n_rows);
    const bool bf16 = layout_param_bf16(layout), l2 = h.mode == ERI_ADAM8_MODE_L2;
    const bool grad_f32 = !layout_grad_bf16(layout);
    const bool wd = h.weight_decay > 0.0f, gs = (h.flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
#define ERI_QE(B, M, W, G) hipLaunchKernelGGL((quant_error_kernel<B, M, W, G>), dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, h, img, dev_scale, err, grad_f32)
#define ERI_QE2(B, M) do { if (wd) { if (gs) ERI_QE(B, M, true, true); else ERI_QE(B, M, true, false); } else { if (gs) ERI_QE(B, M, false, true); else ERI_QE(B, M, false, false); } } while (0)
    if (bf16) { if (l2) ERI_QE2(true, ERI_ADAM8_MODE_L2); else ERI_QE2(true, ERI_ADAM8_MODE_ERI); }
    else { if (l2) ERI_QE2(false, ERI_ADAM8_MODE_L2); else ERI_QE2(false, ERI_ADAM8_MODE_ERI); }
#undef ERI_QE2
#undef ERI_QE
    return (int)hipGetLastError();
}

// ------------------------------------------------------------------------------------------
// plain element-wise sweeps over a row table: 32-bit AdamW and EMA.  One wave per 2048-element
// block, 8 elements per lane and pass, partial last blocks element by element.  HBM-bound:
// AdamW bf16 22 B/param (read 2+2+4+4, write 2+4+4), fp32 28 B/param; EMA 3 x element size.
// ------------------------------------------------------------------------------------------

/* crates/common/optim/src/adamw.rs:34-54, one rounded operation per line */
__device__ __forceinline__ void adamw32_elem(float p, float g, float &m, float &v, const EriAdamW32Hyper &h, float omb1,
                                             float omb2, float neg_lr, float &pn) {
    float ms = m * h.beta1;
    float gs = g * omb1;
    m = ms + gs;
    float vs = v * h.beta2;
    float g2 = g * g;
    float g2s = g2 * omb2;
    v = vs + g2s;
    float denom = sqrtf(v) + h.eps;
    float update = m / denom;
    float wd = h.weight_decay != 0.0f ? p * h.weight_decay : 0.0f;
    float total = update + wd;
    float step = total * neg_lr;
    pn = p + step;
}

template <bool BF16>
__device__ __forceinline__ void store1(void *base, size_t i, float x) {
    if (BF16) as_global(static_cast<uint16_t *>(base))[i] = (uint16_t)bf16_bits(x);
    else as_global(static_cast<float *>(base))[i] = x;
}

/* One full block of the 32-bit step.  MASTER: the parameter value comes from, and goes back to, an fp32
 * master copy; the tensor itself only receives the rounded result (mixed precision,
 * src/kernels/fused_adam.cu:151-193, with the arithmetic of adamw.rs). */
template <bool BF16, bool MASTER, bool GS>
__device__ __forceinline__ void adamw32_block(const ElemRow &t, size_t e0, uint32_t lane, const EriAdamW32Hyper &h,
                                              float omb1, float omb2, float neg_lr, float gscale) {
    char *p = static_cast<char *>(t.a) + e0 * (BF16 ? 2 : 4);
    const char *g = static_cast<const char *>(t.b) + e0 * (BF16 ? 2 : 4);
    float *m = static_cast<float *>(t.c) + e0;
    float *v = static_cast<float *>(t.d) + e0;
    float *w = MASTER ? static_cast<float *>(t.e) + e0 : nullptr;
    Raw8<BF16> pr[4], gr[4];
    Raw8<false> mr[4], vr[4], wr[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t o = c * 512 + lane * 8;
        if (MASTER) wr[c].load(w, o);
        else pr[c].load(p, o);
        gr[c].load(g, o);
        mr[c].load(m, o);
        vr[c].load(v, o);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c) {
        const uint32_t o = c * 512 + lane * 8;
        float pv[8], gv[8], mv[8], vv[8], pn[8];
        if (MASTER) wr[c].unpack(pv);
        else pr[c].unpack(pv);
        gr[c].unpack(gv);
        mr[c].unpack(mv);
        vr[c].unpack(vv);
#pragma unroll
        for (int k = 0; k < 8; ++k) adamw32_elem(pv[k], GS ? gv[k] * gscale : gv[k], mv[k], vv[k], h, omb1, omb2, neg_lr, pn[k]);
        store8<BF16>(p, o, pn);
        if (MASTER) store8<false>(w, o, pn);
        store8<false>(m, o, mv);
        store8<false>(v, o, vv);
    }
}

template <bool BF16, bool GS>
__global__ __launch_bounds__(256) void adamw32_kernel(const ElemRow *__restrict__ rows, uint32_t n_rows,
                                                      uint32_t total_blocks, EriAdamW32Hyper h, float grad_scale,
                                                      const float *__restrict__ dev_scale, uint32_t chunks) {
    // the clip factor left on the device by the gradient-norm pass (1.0 when there is none)
    const float tscale = (GS && dev_scale) ? *dev_scale : 1.0f;
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    const uint32_t stride = gridDim.x * waves_per_wg;
    const float omb1 = 1.0f - h.beta1, omb2 = 1.0f - h.beta2, neg_lr = -h.lr; // adamw.rs:36,42,53
    for (uint32_t r = wave; r < n_rows; r += stride) {
        const ElemRow t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        const size_t e0 = (size_t)(t.numel / kBlock) * kBlock;
        ERI_GLOBAL float *mp = as_global(static_cast<float *>(t.c));
        ERI_GLOBAL float *vp = as_global(static_cast<float *>(t.d));
        ERI_GLOBAL float *wp = as_global(static_cast<float *>(t.e)); // fp32 master copy, or null
        const float gscale = GS ? (grad_scale * t.scale) * tscale : 1.0f; // the order of the 8-bit step's factors
        for (uint32_t i = lane; i < n; i += kWave) {
            float m = mp[e0 + i], v = vp[e0 + i], pn;
            const float pf = wp ? wp[e0 + i] : load1<BF16>(t.a, e0 + i);
            const float gf = load1<BF16>(t.b, e0 + i);
            adamw32_elem(pf, GS ? gf * gscale : gf, m, v, h, omb1, omb2, neg_lr, pn);
            mp[e0 + i] = m;
            vp[e0 + i] = v;
            if (wp) wp[e0 + i] = pn;
            store1<BF16>(t.a, e0 + i, pn);
        }
    }
    uint32_t ti = 0, t_end = 0;
    ElemRow t;
    const BlockWalk walk(total_blocks, chunks);
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        seek_row(rows, n_rows, blk, ti, t, t_end);
        const size_t e0 = (size_t)(blk - t.full_start) * kBlock;
        const float gscale = GS ? (grad_scale * t.scale) * tscale : 1.0f;
        if (t.e) adamw32_block<BF16, true, GS>(t, e0, lane, h, omb1, omb2, neg_lr, gscale);
        else adamw32_block<BF16, false, GS>(t, e0, lane, h, omb1, omb2, neg_lr, gscale);
    }
}

/* src/trainers/ema_enhanced.rs:91-100 */
__device__ __forceinline__ float ema_elem(float shadow, float p, float decay, float omd) {
    float a = shadow * decay;
    float b = p * omd;
    return a + b;
}

template <bool BF16>
__global__ __launch_bounds__(256) void ema_kernel(const ElemRow *__restrict__ rows, uint32_t n_rows,
                                                  uint32_t total_blocks, float decay, uint32_t chunks) {
    const uint32_t lane = threadIdx.x & (kWave - 1);
    const uint32_t waves_per_wg = blockDim.x / kWave;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    const uint32_t stride = gridDim.x * waves_per_wg;
    const float omd = 1.0f - decay; // ema_enhanced.rs:96
    for (uint32_t r = wave; r < n_rows; r += stride) {
        const ElemRow t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        const size_t e0 = (size_t)(t.numel / kBlock) * kBlock;
        for (uint32_t i = lane; i < n; i += kWave)
            store1<BF16>(t.a, e0 + i, ema_elem(load1<BF16>(t.a, e0 + i), load1<BF16>(t.b, e0 + i), decay, omd));
    }
    uint32_t ti = 0, t_end = 0;
    ElemRow t;
    const BlockWalk walk(total_blocks, chunks);
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        seek_row(rows, n_rows, blk, ti, t, t_end);
        const size_t e0 = (size_t)(blk - t.full_start) * kBlock;
        char *s = static_cast<char *>(t.a) + e0 * (BF16 ? 2 : 4);
        const char *p = static_cast<const char *>(t.b) + e0 * (BF16 ? 2 : 4);
        Raw8<BF16> sr[4], pr[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            sr[c].load(s, c * 512 + lane * 8);
            pr[c].load(p, c * 512 + lane * 8);
        }
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            float sv[8], pv[8], out[8];
            sr[c].unpack(sv);
            pr[c].unpack(pv);
#pragma unroll
            for (int k = 0; k < 8; ++k) out[k] = ema_elem(sv[k], pv[k], decay, omd);
            store8<BF16>(s, c * 512 + lane * 8, out);
        }
    }
}

int launch_adamw32(const ElemRow *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag,
                   const EriAdamW32Hyper &h, bool scaled, float grad_scale, const float *dev_scale, uint32_t grid,
                   void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
#define ERI_GO(B, G) hipLaunchKernelGGL((adamw32_kernel<B, G>), dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, h, grad_scale, dev_scale, chunks_for(grid))
    if (dtype_tag == ERI_DTYPE_F32) {
        if (scaled) ERI_GO(false, true);
        else ERI_GO(false, false);
    } else {
        if (scaled) ERI_GO(true, true);
        else ERI_GO(true, false);
    }
#undef ERI_GO
    return (int)hipGetLastError();
}

int launch_ema(const ElemRow *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag, float decay,
               uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype_tag == ERI_DTYPE_F32)
        hipLaunchKernelGGL(ema_kernel<false>, dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, decay, chunks_for(grid));
    else
        hipLaunchKernelGGL(ema_kernel<true>, dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, decay, chunks_for(grid));
    return (int)hipGetLastError();
}

} // namespace eri
