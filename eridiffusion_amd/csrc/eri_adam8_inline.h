#ifndef ERI_ADAM8_INLINE_H
#define ERI_ADAM8_INLINE_H
/*
 * Device code shared by the gfx950 kernels of the blockwise 8-bit AdamW step (everything here is
 * inline or a template; the kernels themselves are in the eri_adam8_*.hip files).
 *
 * Work decomposition: one 64-lane wavefront owns one 2048-element quantisation block from its
 * first load to its last store, so the per-block absmax needs nothing but a DPP reduction inside
 * the wave -- no barrier, no cross-wave exchange.  A block is read in four 512-element passes;
 * lane l of pass c holds elements c*512 + 8*l .. +7, which makes every access a contiguous
 * 128-bit (params, grads) or 64-bit (codes) load per lane.  The fp32 moments of the whole block
 * stay in registers (32 + 32 per lane) between the update and the requantisation, so each byte of
 * p, g, m, v crosses HBM once in each direction.
 *
 * The grid is persistent: workgroups stage the lookup tables into LDS once, then their waves walk
 * the global block list -- cut into one contiguous range per accelerator die, see BlockWalk -- with
 * the stride of their die's waves, so consecutive waves touch consecutive blocks.
 * The tensor that owns a block is found by a scalar binary search over the launch table.
 *
 * Arithmetic: every fp32 operation of the update is written as its own statement and the file is
 * compiled with -ffp-contract=off, because the reference runs each as a separate tensor op
 * (src/trainers/adam8bit_enhanced.rs:252-275).  fmaf appears only inside the exactly rounded
 * division below.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "eri_adam8_device.h"

namespace eri {

// ------------------------------------------------------------------------------------------
// small device helpers
// ------------------------------------------------------------------------------------------

/* Pointers read from the launch table have no known address space; every one of them is device
 * memory, and saying so turns flat_load/flat_store (which also tick the LDS counter and so
 * serialise with the table lookups) into global_load/global_store. */
#define ERI_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ ERI_GLOBAL T *as_global(T *p) {
    return (ERI_GLOBAL T *)p;
}

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t f2u(float x) { return __builtin_bit_cast(uint32_t, x); }
__device__ __forceinline__ float u2f(uint32_t x) { return __builtin_bit_cast(float, x); }

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_mov(float x) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp((int)f2u(x), (int)f2u(x), CTRL, ROW_MASK, 0xf, false));
}

/* Maximum over the 64 lanes of non-negative, NaN-free values, returned wave-uniform.  Such floats
 * order like their bit patterns, so the steps are unsigned integer maxima with the lane permutation
 * folded into the instruction (v_max_u32_dpp); lanes a step does not write keep their value.  A DPP
 * read of a register needs two wait states after the vector instruction that wrote it, and the
 * assembler text below is opaque to the compiler's hazard handling, hence the explicit s_nop. */
#define ERI_DPP_MAX(reg, ctrl) "v_max_u32_dpp " reg ", " reg ", " reg " " ctrl " bank_mask:0xf\n"
__device__ __forceinline__ float wave_max(float x) {
    uint32_t u = f2u(x);
    asm volatile("s_nop 1\n"
                 ERI_DPP_MAX("%0", "quad_perm:[1,0,3,2] row_mask:0xf") "s_nop 1\n"
                 ERI_DPP_MAX("%0", "quad_perm:[2,3,0,1] row_mask:0xf") "s_nop 1\n"
                 ERI_DPP_MAX("%0", "row_half_mirror row_mask:0xf") "s_nop 1\n"
                 ERI_DPP_MAX("%0", "row_mirror row_mask:0xf") "s_nop 1\n" // every lane holds its row's maximum
                 ERI_DPP_MAX("%0", "row_bcast:15 row_mask:0xa") "s_nop 1\n" // into rows 1 and 3
                 ERI_DPP_MAX("%0", "row_bcast:31 row_mask:0xc") "s_nop 1\n" // into rows 2 and 3
                 : "+v"(u));
    return u2f((uint32_t)__builtin_amdgcn_readlane((int)u, 63));
}
/* Two reductions at once: each chain's instruction fills one of the other's wait states. */
__device__ __forceinline__ void wave_max2(float &a, float &b) {
    uint32_t u = f2u(a), w = f2u(b);
#define ERI_DPP_MAX2(ctrl) ERI_DPP_MAX("%0", ctrl) ERI_DPP_MAX("%1", ctrl) "s_nop 0\n"
    asm volatile("s_nop 1\n"
                 ERI_DPP_MAX2("quad_perm:[1,0,3,2] row_mask:0xf")
                 ERI_DPP_MAX2("quad_perm:[2,3,0,1] row_mask:0xf")
                 ERI_DPP_MAX2("row_half_mirror row_mask:0xf")
                 ERI_DPP_MAX2("row_mirror row_mask:0xf")
                 ERI_DPP_MAX2("row_bcast:15 row_mask:0xa")
                 ERI_DPP_MAX2("row_bcast:31 row_mask:0xc")
                 : "+v"(u), "+v"(w));
#undef ERI_DPP_MAX2
    a = u2f((uint32_t)__builtin_amdgcn_readlane((int)u, 63));
    b = u2f((uint32_t)__builtin_amdgcn_readlane((int)w, 63));
}

__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xffff0000u); }

/* fp32 -> bf16 bits, round to nearest even, NaN kept quiet. */
__device__ __forceinline__ uint32_t bf16_bits(float f) {
    __bf16 b = (__bf16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, b);
}
/* Two fp32 -> one dword of two bf16 (lo in the low half): a single v_cvt_pk_bf16_f32. */
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t bf16_pair(float lo, float hi) {
    const f32x2 f = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ float bf16_round(float f) { return u2f(bf16_bits(f) << 16); }

/*
 * SCALE * (m / a) for a divisor shared by a whole block, SCALE a power of two.  With
 * ra = RN(1/a), q0 = RN(m*ra) is within an ulp or two of the quotient, the remainder m - q0*a is
 * exact in one fma, and one correction gives the correctly rounded quotient (Markstein); folding
 * the power of two into ra (and its inverse into a) scales every intermediate exactly.  `fast`
 * excludes the divisors for which that argument needs care (zero, subnormal-range or huge values,
 * an all-ones significand), and those blocks use the hardware-assisted IEEE division instead.
 * Both produce the same bits.
 */
struct BlockDiv {
    float a, as, ras, scale;
    bool fast;
    __device__ __forceinline__ explicit BlockDiv(float a_, float scale_ = 1.0f, float scale_inv = 1.0f)
        : a(a_), scale(scale_) {
        fast = (a_ >= 0x1p-60f) && (a_ <= 0x1p60f) && ((f2u(a_) & 0x7fffffu) != 0x7fffffu);
        const float ra = fast ? 1.0f / a_ : 0.0f;
        ras = ra * scale_;
        as = a_ * scale_inv;
    }
    __device__ __forceinline__ float div_fast(float m) const {
        float q0 = m * ras;
        float r = __builtin_fmaf(-q0, as, m);
        return __builtin_fmaf(r, ras, q0);
    }
    /* div_fast for a numerator that is not tied to the divisor (the bias corrections of the functional
     * update divide moments by 1 - beta^s).  The correction step is exact only while nothing overflows
     * or underflows: an infinite numerator or an overflowing quotient leaves NaN in it, and below
     * 2^-100 the remainder loses bits (one quotient in fifteen then differs from the IEEE result).
     * Those cases take the IEEE division; zero passes through.  Checked on the CPU against IEEE division
     * on 6e8 uniformly random bit patterns and the special values, no difference. */
    __device__ __forceinline__ float div_fast_unbounded(float m) const {
        const float q = div_fast(m);
        const float am = __builtin_fabsf(m), aq = __builtin_fabsf(q);
        const bool ok = aq <= 3.4028234e38f && aq >= 0x1p-100f && am >= 0x1p-100f;
        return ok ? q : (am == 0.0f ? m * scale : m / a * scale);
    }
    __device__ __forceinline__ float div_slow(float m) const {
        float q = a == 0.0f ? 0.0f : m / a;
        return q * scale;
    }
};

struct Lds {
    const float *map_s, *map_u, *mid_s, *mid_u;
    const char *key_s, *key_u;
};

/* Two scaled quotients as binary16 patterns in one dword (a in the low half), rounded toward zero: a single
 * v_cvt_pkrtz_f16_f32.  The slot tables are built for this rounding. */
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t half_key2(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}
__device__ __forceinline__ uint32_t half_key(float xs) { return half_key2(xs, xs) & 0xffffu; }

/* xs = kKeyScale * x.  The slot address is the half pattern with its low bits cleared. */
__device__ __forceinline__ uint32_t code_signed_key(float xs, const char *key_s) {
    const KeySlot s = *reinterpret_cast<const KeySlot *>(key_s + (half_key(xs) & 0xfff0u));
    return s.lo + (xs > s.mid ? 1u : 0u);
}

__device__ __forceinline__ uint32_t code_unsigned_key(float xs, const char *key_u) {
    const KeySlot s = *reinterpret_cast<const KeySlot *>(key_u + (half_key(xs) & 0x7ff8u));
    return s.lo + (xs > s.mid ? 1u : 0u);
}

/* Number of midpoints below x by binary search of the 255-entry LDS table (entry 255 is +inf). */
__device__ __forceinline__ uint32_t code_bsearch(float x, const float *mid) {
    uint32_t idx = 0;
#pragma unroll
    for (uint32_t s = 128; s >= 1; s >>= 1) idx += (x > mid[idx + s - 1]) ? s : 0u;
    return idx;
}

// ------------------------------------------------------------------------------------------
// the update of one element
// ------------------------------------------------------------------------------------------

/* The step's scalars as the kernels use them: the caller's EriAdam8Hyper plus, for the functional update
 * (mode L2), the two constants of its folded fast chain.  That update is
 *     lr * (m / bc1) / (sqrt(v / bc2) + eps)  =  (lr * sqrt(bc2) / bc1) * m / (sqrt(v) + eps * sqrt(bc2)),
 * and the right-hand side needs neither bias correction per element.  Both constants are formed in f64 from the
 * fp32 scalars the exact chain uses and rounded once. */
struct StepHyper : EriAdam8Hyper {
    float l2_step, l2_eps;
    /* The fast chain's error bounds assume a step constant of at most one (so that a normal update means a normal
     * m / denominator) and an eps that swallows the root of a second moment in the denormal range, which the
     * hardware square root does not see.  A launch with other scalars recomputes every element. */
    bool l2_all_exact;
};
template <int MODE>
__device__ __forceinline__ StepHyper make_step_hyper(const EriAdam8Hyper &h) {
    StepHyper s;
    static_cast<EriAdam8Hyper &>(s) = h;
    s.l2_step = 0.0f;
    s.l2_eps = 0.0f;
    s.l2_all_exact = false;
    if (MODE == ERI_ADAM8_MODE_L2) {
        const double root = __builtin_sqrt((double)h.bc2);
        s.l2_step = (float)((double)h.step_size * root / (double)h.bc1);
        s.l2_eps = (float)((double)h.eps * root);
        s.l2_all_exact = !(__builtin_fabsf(s.l2_step) <= 1.0f) || !(s.l2_eps >= 0x1p-36f);
    }
    return s;
}

/* Wave-wide mask of the lanes whose x falls into one of the classes of `classes` (the bits of v_cmp_class_f32):
 * one instruction, where the compiler spells a test for NaN, infinity and denormals as three comparisons. */
__device__ __forceinline__ uint64_t class_mask(float x, uint32_t classes) {
    uint64_t m;
    asm("v_cmp_class_f32 %0, %1, %2" : "=s"(m) : "v"(x), "v"(classes));
    return m;
}

/* The fp32 number halfway between the two bf16 neighbours of x (low half 0x8000): where the rounding of x to
 * bf16 changes direction.  One v_and_or_b32. */
__device__ __forceinline__ float bf16_tie_point(float x) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(f2u(x)), "s"(0xffff0000u), "v"(0x8000u));
    return u2f(r);
}

/* The parameter update from finished moments, one rounded operation per line, with IEEE square root and
 * division: what fp32 parameters always get, and bf16 parameters wherever the fast chain below cannot
 * promise the same bits. */
template <int MODE, bool WD, bool BF16>
__device__ __forceinline__ float param_exact(float p, float m, float v, const StepHyper &h, const BlockDiv &dbc1,
                                             const BlockDiv &dbc2) {
    if (MODE == ERI_ADAM8_MODE_L2) {
        // bf16 parameters come here for one element in 1,600 (the fast chain's near-ties): the plain IEEE
        // division, so that the kernel need not hold the two prepared divisors; fp32 parameters come here
        // with every element and take the prepared form (same bits)
        float mh = BF16 ? m / h.bc1 : dbc1.fast ? dbc1.div_fast_unbounded(m) : m / dbc1.a; // adam8bit.rs:170
        float vh = BF16 ? v / h.bc2 : dbc2.fast ? dbc2.div_fast_unbounded(v) : v / dbc2.a; // :178
        vh = fmaxf(vh, 0.0f);                                           // :181-182
        float den = sqrtf(vh) + h.eps;                                  // :187
        float upd = mh / den;
        float us = upd * h.step_size;  // :196
        if (BF16) us = bf16_round(us); // :197-198: the update is cast to the parameter's dtype
        return p - us;                 // :205
    }
    float den = sqrtf(v) + h.eps; // adam8bit_enhanced.rs:263
    float r = m / den;            // :264
    if (MODE == ERI_ADAM8_MODE_BNB) {
        float us = r * h.step_size;
        float pn = p - us;
        if (WD) pn = pn * h.weight_decay;
        return pn;
    }
    float u = r;
    if (WD) { // :267-271
        float pw = p * h.weight_decay;
        u = r + pw;
    }
    float us = u * h.step_size; // :274
    return p - us;              // :275
}

/*
 * bf16 parameters take the hardware square root and reciprocal (1 ulp each) and two fused multiply-adds
 * instead of the IEEE chain of param_exact, and every element whose bf16 result that could change is
 * flagged through `recheck` (it is only ever set); callers recompute flagged elements with param_exact.
 *
 * Without EXACT (the default arithmetic) the promise is "within one bf16 step of the exact chain".  The
 * approximate chain's error is a few fp32 ulp of the *update*, so it can only exceed a bf16 step of the
 * result where p - update cancels: a result more than 2^12 times smaller than its parameter is flagged
 * (about one element in 10^5 on trained weights).
 *
 * With EXACT the promise is the exact chain's bf16 bits.  Write U = (|r| + |p| wd) * step_size for the size
 * of the update.  Following the roundings of both chains, their results before the last rounding to fp32
 * differ by at most 6.1 * 2^-23 * U (mode BNB: 5.1 * 2^-23 * |r| * step_size, plus one more fp32 rounding
 * each for the decay factor).  Two fp32 values round to the same bf16 value unless a tie point of the bf16
 * grid (the fp32 numbers whose low half is 0x8000) lies between or on them; so if the approximate result
 * pn is further from the tie point T of its own bf16 interval than
 *      margin = 8 * 2^-23 * U  +  |pn| * 2^-22      (the second term is at least two fp32 ulp of pn;
 *                                                     mode BNB: 2^-21, four ulp)
 * the exact chain's fp32 result lies strictly on the same side of T and both round to the same bf16.
 * U is bounded without touching p again: |p| <= |pn| + U (up to roundings), hence
 *      U <= (|r| step_size + wd step_size |pn|) / (1 - wd step_size),
 * which turns the margin into |r| * c_r + |pn| * c_p with two constants of the launch (ExactMargin).
 * Everything else -- about four elements in a million on trained weights, every element whose update
 * cancels its parameter, every NaN or infinity (the comparison is written so that they fail it) -- is
 * flagged.  The slack between 6.1 and 8 covers the use of the approximate r and the rounding of the
 * margin's own arithmetic.
 *
 * The functional update (mode L2) rounds the *update* to bf16 before it subtracts (adam8bit.rs:197-198), and
 * that subtraction is a single exact-input operation, so the same argument applies to the update.  With
 * u = 2^-24: the exact chain rounds m/bc1 (u), v/bc2 (u, halved by the root), the root (u), the sum with eps (u),
 * the quotient (u) and the product with lr (u), 5.5 u in all, relative to the real-valued update.  The fast
 * chain evaluates the folded form (StepHyper): hardware root (2 u), the rounded eps*sqrt(bc2) (u), the sum (u) --
 * the denominator is within 3 u --, the hardware reciprocal (2 u), its product with m (u), the rounded step
 * constant (u) and the last product (u): 8 u.  So the two updates differ by less than 13.5 u = 6.75 * 2^-23 of
 * themselves, which is at most 14 fp32 patterns; an update whose low half is further than kL2TieUlps = 20
 * patterns from 0x8000 rounds to the same bf16 value on both chains.  41 low halves of 65,536 are flagged and
 * recomputed (one element in 1,600), and so is every NaN, infinity and update in the denormal range.
 */
/* v_cmp_class_f32 masks: signalling and quiet NaN, -inf, -denormal, +denormal, +inf. */
constexpr int kClassDenormal = 0x10 | 0x80;
constexpr int kClassNanInfDenormal = 0x1 | 0x2 | 0x4 | 0x200 | kClassDenormal;
/* Mode L2: how close (in fp32 patterns) the low half of the fast chain's update may come to 0x8000 before the
 * element is recomputed.  The two chains' updates differ by less than 6.75 * 2^-23 of themselves (below), which
 * is at most 14 patterns. */
constexpr uint32_t kL2TieUlps = 20;

template <int MODE, bool WD>
struct ExactMargin {
    float c_r, c_p;
    __device__ __forceinline__ explicit ExactMargin(const EriAdam8Hyper &h) {
        constexpr float kEightUlp = 0x1p-20f; // 8 * 2^-23
        if (MODE == ERI_ADAM8_MODE_BNB) {
            c_r = __builtin_fabsf(h.step_size) * kEightUlp;
            c_p = 0x1p-21f;
        } else {
            const float ws = WD ? __builtin_fabsf(h.weight_decay * h.step_size) * 1.001f : 0.0f;
            // a decay that moves a parameter by half of itself per step leaves no bound: flag everything
            const float k = ws < 0.5f ? 1.001f / (1.0f - ws) : __builtin_inff();
            c_r = __builtin_fabsf(h.step_size) * kEightUlp * k;
            c_p = 0x1p-22f + kEightUlp * ws * k;
        }
    }
    __device__ __forceinline__ bool same_bf16_as_exact(float r, float pn) const {
        // the floor 2^-126 flags everything down among the fp32 denormals, where the bounds above do not hold
        const float margin = __builtin_fmaf(__builtin_fabsf(pn), c_p, __builtin_fmaf(__builtin_fabsf(r), c_r, 0x1p-126f));
        return __builtin_fabsf(pn - bf16_tie_point(pn)) > margin;
    }
};

/* Which lanes must recompute which of their eight elements with param_exact: one wave-wide mask per position,
 * held in scalar registers.  (As an array of per-lane bools the flags were materialised in vector registers:
 * three vector instructions per element.)  A position no lane has flagged is skipped altogether. */
struct Redo8 {
    uint64_t lanes[8];
    uint64_t any;
    __device__ __forceinline__ Redo8() : any(0) {}
    __device__ __forceinline__ void set(int k, uint64_t flagged) {
        lanes[k] = flagged;
        any |= flagged;
    }
    /* every active lane recomputes all of its elements */
    __device__ __forceinline__ void set_all() {
        const uint64_t active = __builtin_amdgcn_ballot_w64(true);
        for (int k = 0; k < 8; ++k) lanes[k] = active;
        any = active;
    }
    __device__ __forceinline__ bool mine(int k) const { return __builtin_amdgcn_inverse_ballot_w64(lanes[k]); }
};

/* t1 = m_old * beta1 and t3 = v_old * beta2 come in already multiplied: a kernel that holds a block's 256
 * possible values of either product in a table of its own forms them once per code instead of once per
 * element (same two rounded multiplications, same bits). */
template <int MODE, bool EXACT, bool BF16, bool WD, bool GS>
__device__ __forceinline__ void adam_elem_decayed(float p, float g, float t1, float t3, const StepHyper &h,
                                                  float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, float &m,
                                                  float &v, float &pn, uint64_t &recheck);

template <int MODE, bool EXACT, bool BF16, bool WD, bool GS>
__device__ __forceinline__ void adam_elem(float p, float g, float m_old, float v_old, const StepHyper &h,
                                          float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, float &m,
                                          float &v, float &pn, uint64_t &recheck) {
    float t1 = m_old * h.beta1; // adam8bit_enhanced.rs:256
    float t3 = v_old * h.beta2; // :260
    adam_elem_decayed<MODE, EXACT, BF16, WD, GS>(p, g, t1, t3, h, gscale, dbc1, dbc2, m, v, pn, recheck);
}

template <int MODE, bool EXACT, bool BF16, bool WD, bool GS>
__device__ __forceinline__ void adam_elem_decayed(float p, float g, float t1, float t3, const StepHyper &h,
                                                  float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, float &m,
                                                  float &v, float &pn, uint64_t &recheck) {
    if (GS) g = g * gscale;
    if (MODE == ERI_ADAM8_MODE_L2 && WD) { // adam8bit.rs:113-120
        float pw = p * h.weight_decay;
        g = g + pw;
    }
    float t2 = g * h.omb1; // adam8bit_enhanced.rs:256
    m = t1 + t2;
    float gg = g * g; // :259-260
    float t4 = gg * h.omb2;
    v = t3 + t4;
    if (!BF16) { // fp32 parameters: every bit of the exact chain counts
        pn = param_exact<MODE, WD, false>(p, m, v, h, dbc1, dbc2);
    } else if (MODE == ERI_ADAM8_MODE_L2) { // always to the exact chain's bits (the reference rounds the update itself)
        // fast chain: the folded form of the update (StepHyper), hardware square root and reciprocal;
        // param_exact redoes whatever the tests below cannot vouch for
        float den = __builtin_amdgcn_sqrtf(v) + h.l2_eps;
        float r = m * __builtin_amdgcn_rcpf(den);
        float us = r * h.l2_step;
        // Both chains round the update to bf16, so they agree unless a rounding boundary of bf16 (an fp32 pattern
        // whose low half is 0x8000) lies between their updates, and those are at most 14 fp32 patterns apart
        // (kL2TieUlps covers it with room): flagged are the updates whose low half is that close to 0x8000.
        const uint32_t moved = f2u(us) + (kL2TieUlps - 0x8000u);
        recheck |= __builtin_amdgcn_ballot_w64((moved & 0xffffu) <= 2u * kL2TieUlps);
        // NaN, infinity and updates in the denormal range, where the relative bounds do not hold (a zero
        // update is a zero moment on both chains and passes).  Launches whose scalars void the bounds altogether
        // (StepHyper::l2_all_exact) recompute every element: the kernels see to that, not this chain.
        recheck |= class_mask(us, kClassNanInfDenormal);
        pn = p - u2f(bf16_pair(0.0f, us)); // adam8bit.rs:197-205: the update rounded to bf16, then subtracted
    } else { // h.eps and h.weight_decay of mode BNB carry sqrt(bc2) and the factor 1 - lr*wd
        float den = __builtin_amdgcn_sqrtf(v) + h.eps;
        float r = m * __builtin_amdgcn_rcpf(den);
        if (MODE == ERI_ADAM8_MODE_BNB) {
            float p0 = __builtin_fmaf(-r, h.step_size, p);
            pn = WD ? p0 * h.weight_decay : p0;
            if (EXACT) recheck |= __builtin_amdgcn_ballot_w64(!ExactMargin<MODE, WD>(h).same_bf16_as_exact(r, pn));
            else recheck |= __builtin_amdgcn_ballot_w64(__builtin_fabsf(p0) * 4096.0f < __builtin_fabsf(p));
        } else {
            float u = WD ? __builtin_fmaf(p, h.weight_decay, r) : r;
            pn = __builtin_fmaf(-u, h.step_size, p);
            if (EXACT) recheck |= __builtin_amdgcn_ballot_w64(!ExactMargin<MODE, WD>(h).same_bf16_as_exact(r, pn));
            else recheck |= __builtin_amdgcn_ballot_w64(__builtin_fabsf(pn) * 4096.0f < __builtin_fabsf(p));
        }
    }
}

// ------------------------------------------------------------------------------------------
// 8 consecutive elements per lane: loads and stores
// ------------------------------------------------------------------------------------------

/* Eight consecutive elements of one lane as they come from memory: one 128-bit word of bf16, or
 * two of fp32.  Loading and unpacking are separate so that a block's loads can all be issued
 * before the first value is needed. */
template <bool BF16>
struct Raw8;
template <>
struct Raw8<true> {
    u32x4 w;
    __device__ __forceinline__ void load(const void *base, uint32_t elem) {
        // every byte these kernels stream is touched once per launch: non-temporal throughout
        w = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(base) + elem)));
    }
    __device__ __forceinline__ void unpack(float (&out)[8]) const {
        out[0] = bf16_lo(w.x); out[1] = bf16_hi(w.x); out[2] = bf16_lo(w.y); out[3] = bf16_hi(w.y);
        out[4] = bf16_lo(w.z); out[5] = bf16_hi(w.z); out[6] = bf16_lo(w.w); out[7] = bf16_hi(w.w);
    }
};
template <>
struct Raw8<false> {
    f32x4 a, b;
    __device__ __forceinline__ void load(const void *base, uint32_t elem) {
        ERI_GLOBAL const f32x4 *q = as_global(reinterpret_cast<const f32x4 *>(static_cast<const float *>(base) + elem));
        // a lane's two words share cache lines with its neighbours' across the two instructions, so these
        // stay ordinary loads: streamed, the second instruction would fetch every line again
        a = q[0];
        b = q[1];
    }
    __device__ __forceinline__ void unpack(float (&out)[8]) const {
        out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w;
        out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
    }
};

template <bool BF16>
__device__ __forceinline__ void store8(void *base, uint32_t elem, const float (&v)[8]) {
    if (BF16) {
        u32x4 w;
        w.x = bf16_pair(v[0], v[1]);
        w.y = bf16_pair(v[2], v[3]);
        w.z = bf16_pair(v[4], v[5]);
        w.w = bf16_pair(v[6], v[7]);
        __builtin_nontemporal_store(w, as_global(reinterpret_cast<u32x4 *>(static_cast<uint16_t *>(base) + elem)));
    } else {
        ERI_GLOBAL f32x4 *q = as_global(reinterpret_cast<f32x4 *>(static_cast<float *>(base) + elem));
        q[0] = f32x4{v[0], v[1], v[2], v[3]}; // half a line per instruction: left to the cache to merge
        q[1] = f32x4{v[4], v[5], v[6], v[7]};
    }
}

__device__ __forceinline__ uint32_t byte_of(const u32x2 w, int k) {
    const uint32_t d = k < 4 ? w.x : w.y;
    return (d >> (8 * (k & 3))) & 0xffu;
}

/* 4 * (byte k of the eight packed codes): the LDS byte offset of a float table entry, in one
 * sub-dword-addressed shift (v_lshlrev_b32 with an SDWA byte select) instead of an extract and a
 * shift.  k must be a compile-time constant after unrolling. */
__device__ __forceinline__ uint32_t code_offset(const u32x2 w, int k) {
    const uint32_t d = k < 4 ? w.x : w.y;
    const uint32_t two = 2u;
    uint32_t r;
    switch (k & 3) {
    case 0:
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(two), "v"(d));
        break;
    case 1:
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(two), "v"(d));
        break;
    case 2:
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(two), "v"(d));
        break;
    default:
        asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(two), "v"(d));
        break;
    }
    return r;
}
__device__ __forceinline__ float lds_float_at(const float *table, uint32_t byte_offset) {
    return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(table) + byte_offset);
}

// ------------------------------------------------------------------------------------------
// a full 2048-element block, one wavefront
// ------------------------------------------------------------------------------------------

/*
 * acc.byte[k] = lo + (xs > mid): the compare, the add and the insertion into the packed word of four
 * codes in two instructions -- a carry-in add whose SDWA destination select writes one byte and
 * preserves the others.  Every block opens with the compare, so two byte writes into the same
 * register are never adjacent (the sub-dword write needs one instruction before its result is
 * read); the last byte is followed by an s_nop before the store consumes the word.
 * k must be a compile-time constant after unrolling.
 */
__device__ __forceinline__ void pack_code(uint32_t &acc, int k, float xs, float mid, uint32_t lo) {
    const uint32_t zero = 0u;
    switch (k & 3) {
    case 0:
        asm("v_cmp_gt_f32 vcc, %1, %2\n\t"
            "v_addc_co_u32_sdwa %0, vcc, %3, %4, vcc dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD"
            : "=v"(acc) : "v"(xs), "v"(mid), "v"(lo), "v"(zero) : "vcc");
        break;
    case 1:
        asm("v_cmp_gt_f32 vcc, %1, %2\n\t"
            "v_addc_co_u32_sdwa %0, vcc, %3, %4, vcc dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
            : "+v"(acc) : "v"(xs), "v"(mid), "v"(lo), "v"(zero) : "vcc");
        break;
    case 2:
        asm("v_cmp_gt_f32 vcc, %1, %2\n\t"
            "v_addc_co_u32_sdwa %0, vcc, %3, %4, vcc dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD"
            : "+v"(acc) : "v"(xs), "v"(mid), "v"(lo), "v"(zero) : "vcc");
        break;
    default:
        asm("v_cmp_gt_f32 vcc, %1, %2\n\t"
            "v_addc_co_u32_sdwa %0, vcc, %3, %4, vcc dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD\n\t"
            "s_nop 0"
            : "+v"(acc) : "v"(xs), "v"(mid), "v"(lo), "v"(zero) : "vcc");
        break;
    }
}

/* Mode BNB: a first-moment code whose map value has the other sign than the moment moves one entry
 * toward the moment's sign.  The signed map is negative below entry 127, zero at 127 and positive
 * above, and the quotient has the moment's sign, so the only case is a negative moment that
 * rounds to the zero entry: it takes entry 126, the negative value nearest zero. */
__device__ __forceinline__ uint32_t keep_sign(uint32_t code, float m, float absmax) {
    return (code == 127u && (f2u(m) >> 31) != 0u && absmax != 0.0f) ? 126u : code;
}

template <bool FAST_DIV, bool KEYTAB, bool KEEP_SIGN = false>
__device__ __forceinline__ void requant8(const float *mf, const float *vf, const BlockDiv &dm, const BlockDiv &dv,
                                         const Lds &L, u32x2 &mw, u32x2 &vw) {
    if (KEYTAB && FAST_DIV && !KEEP_SIGN) { // the hot path: slot lookup, codes packed by byte-select writes
        uint32_t am[2], av[2];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const float xm = dm.div_fast(mf[k]); // times kKeyScale
            const float xv = dv.div_fast(vf[k]);
            const uint32_t keys = half_key2(xm, xv); // both slot addresses out of one conversion
            const KeySlot sm = *reinterpret_cast<const KeySlot *>(L.key_s + (keys & 0xfff0u));
            const KeySlot sv = *reinterpret_cast<const KeySlot *>(L.key_u + ((keys >> 16) & 0x7ff8u));
            pack_code(am[k >> 2], k, xm, sm.mid, sm.lo);
            pack_code(av[k >> 2], k, xv, sv.mid, sv.lo);
        }
        mw.x = am[0]; mw.y = am[1];
        vw.x = av[0]; vw.y = av[1];
        return;
    }
    uint32_t cm[8], cv[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float xm = FAST_DIV ? dm.div_fast(mf[k]) : dm.div_slow(mf[k]); // times dm.scale
        const float xv = FAST_DIV ? dv.div_fast(vf[k]) : dv.div_slow(vf[k]);
        cm[k] = KEYTAB ? code_signed_key(xm, L.key_s) : code_bsearch(xm, L.mid_s);
        if (KEEP_SIGN) cm[k] = keep_sign(cm[k], mf[k], dm.a);
        cv[k] = KEYTAB ? code_unsigned_key(xv, L.key_u) : code_bsearch(xv, L.mid_u);
    }
    mw.x = cm[0] | (cm[1] << 8) | (cm[2] << 16) | (cm[3] << 24);
    mw.y = cm[4] | (cm[5] << 8) | (cm[6] << 16) | (cm[7] << 24);
    vw.x = cv[0] | (cv[1] << 8) | (cv[2] << 16) | (cv[3] << 24);
    vw.y = cv[4] | (cv[5] << 8) | (cv[6] << 16) | (cv[7] << 24);
}

/* `mine` is the wave's own pair of 256-entry tables in LDS.  The block opens by filling them with
 * (MAP[c] * absmax) * beta for every code c -- the first two operations of both moment updates, done once
 * per code (eight per lane) instead of once per element (64 per lane); a wave's LDS operations complete in
 * order, so its reads below see its own writes without a barrier. */
template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB, bool GBF16 = BF16>
__device__ __forceinline__ void full_block(const DevTensor &t, uint32_t lb, uint32_t lane, const StepHyper &h,
                                           float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, const Lds &L,
                                           float (*mine)[256]) {
    const size_t e0 = (size_t)lb * kBlock;
    const size_t esz = BF16 ? 2 : 4;
    char *p = static_cast<char *>(t.p) + e0 * esz;
    const char *p_in = static_cast<const char *>(t.p_in) + e0 * esz;
    const char *g = static_cast<const char *>(t.g) + e0 * (GBF16 ? 2 : 4);
    uint8_t *mc = t.m + e0;
    uint8_t *vc = t.v + e0;
    const float a_m = as_global(t.absmax_m)[lb];
    const float a_v = as_global(t.absmax_v)[lb];
    {
        const f32x4 bs = reinterpret_cast<const f32x4 *>(L.map_s)[lane]; // codes 4*lane .. 4*lane + 3
        const f32x4 bu = reinterpret_cast<const f32x4 *>(L.map_u)[lane];
        f32x4 ds, du;
        ds.x = (bs.x * a_m) * h.beta1; ds.y = (bs.y * a_m) * h.beta1;
        ds.z = (bs.z * a_m) * h.beta1; ds.w = (bs.w * a_m) * h.beta1;
        du.x = (bu.x * a_v) * h.beta2; du.y = (bu.y * a_v) * h.beta2;
        du.z = (bu.z * a_v) * h.beta2; du.w = (bu.w * a_v) * h.beta2;
        reinterpret_cast<f32x4 *>(mine[0])[lane] = ds;
        reinterpret_cast<f32x4 *>(mine[1])[lane] = du;
    }

    float mf[32], vf[32];
    float lm = 0.0f, lv = 0.0f;
    // Issue the loads of DEPTH passes before touching the first value: the wave then waits once per
    // DEPTH passes, with 48 * DEPTH bytes per lane in flight (bf16; fp32 values hold twice the registers).
    constexpr int DEPTH = (BF16 && GBF16) ? 4 : 2;
#pragma unroll
    for (int c0 = 0; c0 < 4; c0 += DEPTH) {
        Raw8<BF16> pr[DEPTH];
        Raw8<GBF16> gr[DEPTH];
        u32x2 mr[DEPTH], vr[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const uint32_t o = (c0 + d) * 512 + lane * 8;
            pr[d].load(p_in, o);
            gr[d].load(g, o);
            mr[d] = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x2 *>(mc + o)));
            vr[d] = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x2 *>(vc + o)));
        }
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const int c = c0 + d;
            const uint32_t o = c * 512 + lane * 8;
            float pv[8], gv[8], pn[8];
            pr[d].unpack(pv);
            gr[d].unpack(gv);
            // one flag per element: the exact chain then runs for the flagged positions only
            Redo8 redo;
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float t1 = lds_float_at(mine[0], code_offset(mr[d], k));
                const float t3 = lds_float_at(mine[1], code_offset(vr[d], k));
                float m, v;
                uint64_t flagged = 0;
                adam_elem_decayed<MODE, EXACT, BF16, WD, GS>(pv[k], gv[k], t1, t3, h, gscale, dbc1, dbc2, m, v, pn[k], flagged);
                redo.set(k, flagged);
                mf[c * 8 + k] = m;
                vf[c * 8 + k] = v;
                lm = fmaxf(lm, __builtin_fabsf(m));
                lv = fmaxf(lv, __builtin_fabsf(v));
            }
            if (BF16 && MODE == ERI_ADAM8_MODE_L2 && h.l2_all_exact) redo.set_all();
            if (BF16 && redo.any) {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (redo.lanes[k] && redo.mine(k))
                        pn[k] = param_exact<MODE, WD, BF16>(pv[k], mf[c * 8 + k], vf[c * 8 + k], h, dbc1, dbc2);
            }
            store8<BF16>(p, o, pn);
        }
    }
    float nam = lm, nav = lv;
    wave_max2(nam, nav);
    if (lane == 0) {
        as_global(t.absmax_m)[lb] = nam;
        as_global(t.absmax_v)[lb] = nav;
    }
    constexpr float ks = KEYTAB ? kKeyScale : 1.0f, ksi = KEYTAB ? kKeyScaleInv : 1.0f;
    const BlockDiv dm(nam, ks, ksi), dv(nav, ks, ksi);
    if (dm.fast && dv.fast) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t o = c * 512 + lane * 8;
            u32x2 mw, vw;
            requant8<true, KEYTAB, MODE == ERI_ADAM8_MODE_BNB>(mf + c * 8, vf + c * 8, dm, dv, L, mw, vw);
            __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(mc + o)));
            __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(vc + o)));
        }
    } else {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t o = c * 512 + lane * 8;
            u32x2 mw, vw;
            requant8<false, KEYTAB, MODE == ERI_ADAM8_MODE_BNB>(mf + c * 8, vf + c * 8, dm, dv, L, mw, vw);
            __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(mc + o)));
            __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(vc + o)));
        }
    }
}

// ------------------------------------------------------------------------------------------
// the last, partial block of a tensor: element-wise, bounds-checked, moments recomputed in the
// second sweep instead of being held (n < 2048 elements, once per tensor at most)
// ------------------------------------------------------------------------------------------

template <bool BF16>
__device__ __forceinline__ float load1(const void *base, size_t i) {
    if (BF16) return u2f((uint32_t)as_global(static_cast<const uint16_t *>(base))[i] << 16);
    return as_global(static_cast<const float *>(base))[i];
}

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB, bool GBF16 = BF16>
__device__ __forceinline__ void tail_block(const DevTensor &t, uint32_t lb, uint32_t n, uint32_t lane,
                                        const StepHyper &h, float gscale, const BlockDiv &dbc1,
                                        const BlockDiv &dbc2, const Lds &L) {
    const size_t e0 = (size_t)lb * kBlock;
    ERI_GLOBAL uint8_t *mc = as_global(t.m);
    ERI_GLOBAL uint8_t *vc = as_global(t.v);
    const float a_m = as_global(t.absmax_m)[lb];
    const float a_v = as_global(t.absmax_v)[lb];
    float lm = 0.0f, lv = 0.0f;
    constexpr float ks = KEYTAB ? kKeyScale : 1.0f, ksi = KEYTAB ? kKeyScaleInv : 1.0f;
    if ((n & 7u) == 0) {
        // The usual case (tensor sizes are multiples of eight): the same 8-elements-per-lane accesses as a
        // full block, lanes past the end switched off.  Two sweeps, the second recomputing the moments,
        // so that nothing but one pass of values is held -- this code is inlined into kernels whose
        // register budget belongs to their main loop.
        const size_t esz = BF16 ? 2 : 4;
        char *p = static_cast<char *>(t.p) + e0 * esz;
        const char *p_in = static_cast<const char *>(t.p_in) + e0 * esz;
        const char *g = static_cast<const char *>(t.g) + e0 * (GBF16 ? 2 : 4);
        const uint32_t passes = (n + 511) / 512;
        for (uint32_t c = 0; c < passes; ++c) {
            const uint32_t o = c * 512 + lane * 8;
            if (o < n) {
                Raw8<BF16> pr;
                Raw8<GBF16> gr;
                pr.load(p_in, o);
                gr.load(g, o);
                const u32x2 mr = *as_global(reinterpret_cast<const u32x2 *>(t.m + e0 + o));
                const u32x2 vr = *as_global(reinterpret_cast<const u32x2 *>(t.v + e0 + o));
                float pv[8], gv[8];
                pr.unpack(pv);
                gr.unpack(gv);
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    float m, v, pn;
                    uint64_t unused = 0;
                    adam_elem<MODE, EXACT, BF16, WD, GS>(pv[k], gv[k], L.map_s[byte_of(mr, k)] * a_m,
                                                         L.map_u[byte_of(vr, k)] * a_v, h, gscale, dbc1, dbc2, m, v, pn, unused);
                    lm = fmaxf(lm, __builtin_fabsf(m));
                    lv = fmaxf(lv, __builtin_fabsf(v));
                }
            }
        }
        float nam = lm, nav = lv;
        wave_max2(nam, nav);
        const BlockDiv dm(nam, ks, ksi), dv(nav, ks, ksi);
        for (uint32_t c = 0; c < passes; ++c) {
            const uint32_t o = c * 512 + lane * 8;
            if (o < n) {
                Raw8<BF16> pr;
                Raw8<GBF16> gr;
                pr.load(p_in, o);
                gr.load(g, o);
                const u32x2 mr = *as_global(reinterpret_cast<const u32x2 *>(t.m + e0 + o));
                const u32x2 vr = *as_global(reinterpret_cast<const u32x2 *>(t.v + e0 + o));
                float pv[8], gv[8], pn[8], m[8], v[8];
                pr.unpack(pv);
                gr.unpack(gv);
                uint64_t cancel = (BF16 && MODE == ERI_ADAM8_MODE_L2 && h.l2_all_exact) ? ~0ull : 0ull;
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    adam_elem<MODE, EXACT, BF16, WD, GS>(pv[k], gv[k], L.map_s[byte_of(mr, k)] * a_m,
                                                         L.map_u[byte_of(vr, k)] * a_v, h, gscale, dbc1, dbc2, m[k], v[k], pn[k], cancel);
                if (BF16 && __builtin_amdgcn_inverse_ballot_w64(cancel)) { // a lane with a flagged element redoes its eight
#pragma unroll
                    for (int k = 0; k < 8; ++k) pn[k] = param_exact<MODE, WD, BF16>(pv[k], m[k], v[k], h, dbc1, dbc2);
                }
                u32x2 mw, vw;
                requant8<false, KEYTAB, MODE == ERI_ADAM8_MODE_BNB>(m, v, dm, dv, L, mw, vw);
                *as_global(reinterpret_cast<u32x2 *>(t.m + e0 + o)) = mw;
                *as_global(reinterpret_cast<u32x2 *>(t.v + e0 + o)) = vw;
                store8<BF16>(p, o, pn);
            }
        }
        if (lane == 0) {
            as_global(t.absmax_m)[lb] = nam;
            as_global(t.absmax_v)[lb] = nav;
        }
        return;
    }
    for (uint32_t i = lane; i < n; i += kWave) {
        const size_t e = e0 + i;
        float m, v, pn;
        uint64_t unused = 0;
        adam_elem<MODE, EXACT, BF16, WD, GS>(load1<BF16>(t.p_in, e), load1<GBF16>(t.g, e), L.map_s[mc[e]] * a_m,
                                             L.map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn, unused);
        lm = fmaxf(lm, __builtin_fabsf(m));
        lv = fmaxf(lv, __builtin_fabsf(v));
    }
    float nam = lm, nav = lv;
    wave_max2(nam, nav);
    const BlockDiv dm(nam, ks, ksi), dv(nav, ks, ksi);
    for (uint32_t i = lane; i < n; i += kWave) {
        const size_t e = e0 + i;
        float m, v, pn;
        uint64_t cancel = (BF16 && MODE == ERI_ADAM8_MODE_L2 && h.l2_all_exact) ? ~0ull : 0ull;
        const float p_old = load1<BF16>(t.p_in, e);
        adam_elem<MODE, EXACT, BF16, WD, GS>(p_old, load1<GBF16>(t.g, e), L.map_s[mc[e]] * a_m,
                                             L.map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn, cancel);
        if (BF16 && __builtin_amdgcn_inverse_ballot_w64(cancel)) pn = param_exact<MODE, WD, BF16>(p_old, m, v, h, dbc1, dbc2);
        const float xm = dm.div_slow(m);
        const float xv = dv.div_slow(v);
        uint32_t cm = KEYTAB ? code_signed_key(xm, L.key_s) : code_bsearch(xm, L.mid_s);
        if (MODE == ERI_ADAM8_MODE_BNB) cm = keep_sign(cm, m, nam);
        mc[e] = (uint8_t)cm;
        vc[e] = (uint8_t)(KEYTAB ? code_unsigned_key(xv, L.key_u) : code_bsearch(xv, L.mid_u));
        if (BF16) as_global(static_cast<uint16_t *>(t.p))[e] = (uint16_t)bf16_bits(pn);
        else as_global(static_cast<float *>(t.p))[e] = pn;
    }
    if (lane == 0) {
        as_global(t.absmax_m)[lb] = nam;
        as_global(t.absmax_v)[lb] = nav;
    }
}

// ------------------------------------------------------------------------------------------
// the step kernel
// ------------------------------------------------------------------------------------------

/* The table image, staged once per workgroup.  A static array: its LDS address is a compile-time
 * constant, so table offsets fold into the ds_read immediates. */
#define ERI_LDS_IMAGE __shared__ uint4 lds_raw[kLdsImageBytes / 16]

/* Row owning full block `blk`: the last row whose full_start is <= blk (rows without full blocks
 * share their successor's full_start and are skipped by taking the last).  All wave-uniform. */
template <typename Row>
__device__ __forceinline__ uint32_t find_row(const Row *rows, uint32_t n_rows, uint32_t from, uint32_t blk) {
    uint32_t lo = from, hi = n_rows; // rows[lo].full_start <= blk
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (rows[mid].full_start <= blk) lo = mid; else hi = mid;
    }
    return lo;
}

/* A wave's blocks only grow and a tensor usually spans many of them, so the owning row is looked up
 * again only when a block leaves the range [t.full_start, t_end) of the row at hand (t_end = 0 forces
 * the first lookup).  A launch table carries, right behind its rows, one row index per full block
 * (BlockRowMap): the lookup is then one scalar load and the load of the row, where the search takes ten
 * dependent loads -- which a table of many small tensors pays on almost every block, because a wave's
 * consecutive blocks lie a whole stride apart.  Row tables without the map (the plain element-wise sweeps)
 * search. */
template <typename Row>
__device__ __forceinline__ void seek_row(const Row *rows, uint32_t n_rows, uint32_t blk, uint32_t &ti, Row &t,
                                         uint32_t &t_end) {
    if (blk >= t_end) {
        ti = find_row(rows, n_rows, ti, blk);
        t = rows[ti];
        t_end = t.full_start + (uint32_t)(t.numel / kBlock);
    }
}

struct BlockRowMap {
    const uint32_t *row_of; // row_of[b] = index of the row that owns full block b
    __device__ __forceinline__ BlockRowMap(const DevTensor *rows, uint32_t n_rows)
        : row_of(reinterpret_cast<const uint32_t *>(rows + n_rows)) {}
    __device__ __forceinline__ void seek(const DevTensor *rows, uint32_t blk, uint32_t &ti, DevTensor &t, uint32_t &t_end) const {
        if (blk >= t_end) {
            ti = row_of[blk];
            t = rows[ti];
            t_end = t.full_start + (uint32_t)(t.numel / kBlock);
        }
    }
};

/* The full blocks one wave walks.  Workgroup i of a launch runs on accelerator die (XCD) i mod 8.  The
 * block list is cut into `chunks` contiguous ranges and workgroup i walks range i mod chunks, so with
 * chunks == 8 each die sweeps its own part of every buffer instead of all dies advancing through one
 * common window; on MI355X that made the sweep both a little faster and much less dependent on where
 * the buffers happen to lie physically.  chunks == 1 is the plain grid-stride walk. */
struct BlockWalk {
    uint32_t first, end, stride;
    __device__ __forceinline__ BlockWalk(uint32_t total_blocks, uint32_t chunks) {
        const uint32_t waves_per_wg = blockDim.x / kWave;
        const uint32_t per_chunk = (total_blocks + chunks - 1) / chunks;
        const uint32_t lo = (blockIdx.x % chunks) * per_chunk;
        end = lo + per_chunk < total_blocks ? lo + per_chunk : total_blocks;
        stride = (gridDim.x / chunks) * waves_per_wg;
        first = __builtin_amdgcn_readfirstlane(lo + (blockIdx.x / chunks) * waves_per_wg + threadIdx.x / kWave);
    }
};


} // namespace eri
#endif /* ERI_ADAM8_INLINE_H */
