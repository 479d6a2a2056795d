/*
 * gfx950 kernels of the blockwise 8-bit AdamW step.
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

__device__ __forceinline__ uint32_t half_key(float xs) {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)xs); // v_cvt_f16_f32, round to nearest even
}

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

template <int MODE, bool EXACT, bool BF16, bool WD, bool GS>
__device__ __forceinline__ void adam_elem(float p, float g, float m_old, float v_old, const EriAdam8Hyper &h,
                                          float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, float &m,
                                          float &v, float &pn) {
    if (GS) g = g * gscale;
    if (MODE == ERI_ADAM8_MODE_L2 && WD) { // adam8bit.rs:113-120
        float pw = p * h.weight_decay;
        g = g + pw;
    }
    float t1 = m_old * h.beta1; // adam8bit_enhanced.rs:256
    float t2 = g * h.omb1;
    m = t1 + t2;
    float gg = g * g; // :259-260
    float t3 = v_old * h.beta2;
    float t4 = gg * h.omb2;
    v = t3 + t4;
    if (MODE == ERI_ADAM8_MODE_L2) {
        float mh = dbc1.fast ? dbc1.div_fast_unbounded(m) : m / dbc1.a; // adam8bit.rs:170
        float vh = dbc2.fast ? dbc2.div_fast_unbounded(v) : v / dbc2.a; // :178
        vh = fmaxf(vh, 0.0f);                                  // :181-182
        float upd;
        if (EXACT) {
            float den = sqrtf(vh) + h.eps; // :187
            upd = mh / den;
        } else {
            float den = __builtin_amdgcn_sqrtf(vh) + h.eps;
            upd = mh * __builtin_amdgcn_rcpf(den);
        }
        float us = upd * h.step_size; // :196
        if (BF16) us = bf16_round(us); // :197-198
        pn = p - us;                   // :205
    } else if (MODE == ERI_ADAM8_MODE_BNB) { // h.eps carries sqrt(bc2), h.weight_decay is the factor 1 - lr*wd
        float den = sqrtf(v) + h.eps;
        float r = m / den;
        float us = r * h.step_size;
        pn = p - us;
        if (WD) pn = pn * h.weight_decay;
    } else {
        if (EXACT) {
            float den = sqrtf(v) + h.eps; // adam8bit_enhanced.rs:263
            float r = m / den;            // :264
            float u = r;
            if (WD) { // :267-271
                float pw = p * h.weight_decay;
                u = r + pw;
            }
            float us = u * h.step_size; // :274
            pn = p - us;                // :275
        } else {
            // bf16 parameters: hardware square root and reciprocal (1 ulp each) and two fused
            // multiply-adds; the fp32 result is within a few ulp of the exact chain, which moves
            // the bf16 rounding of p by at most one step, rarely
            float den = __builtin_amdgcn_sqrtf(v) + h.eps;
            float r = m * __builtin_amdgcn_rcpf(den);
            float u = WD ? __builtin_fmaf(p, h.weight_decay, r) : r;
            pn = __builtin_fmaf(-u, h.step_size, p);
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
            const KeySlot sm = *reinterpret_cast<const KeySlot *>(L.key_s + (half_key(xm) & 0xfff0u));
            const KeySlot sv = *reinterpret_cast<const KeySlot *>(L.key_u + (half_key(xv) & 0x7ff8u));
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

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB>
__device__ __forceinline__ void full_block(const DevTensor &t, uint32_t lb, uint32_t lane, const EriAdam8Hyper &h,
                                           float gscale, const BlockDiv &dbc1, const BlockDiv &dbc2, const Lds &L) {
    const size_t e0 = (size_t)lb * kBlock;
    const size_t esz = BF16 ? 2 : 4;
    char *p = static_cast<char *>(t.p) + e0 * esz;
    const char *g = static_cast<const char *>(t.g) + e0 * esz;
    uint8_t *mc = t.m + e0;
    uint8_t *vc = t.v + e0;
    const float a_m = as_global(t.absmax_m)[lb];
    const float a_v = as_global(t.absmax_v)[lb];

    float mf[32], vf[32];
    float lm = 0.0f, lv = 0.0f;
    // Issue the loads of DEPTH passes before touching the first value: the wave then waits once per
    // DEPTH passes, with 48 * DEPTH bytes per lane in flight (bf16; fp32 holds twice the registers).
    constexpr int DEPTH = BF16 ? 4 : 2;
#pragma unroll
    for (int c0 = 0; c0 < 4; c0 += DEPTH) {
        Raw8<BF16> pr[DEPTH], gr[DEPTH];
        u32x2 mr[DEPTH], vr[DEPTH];
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const uint32_t o = (c0 + d) * 512 + lane * 8;
            pr[d].load(p, o);
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
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float m_old = L.map_s[byte_of(mr[d], k)] * a_m;
                const float v_old = L.map_u[byte_of(vr[d], k)] * a_v;
                float m, v;
                adam_elem<MODE, EXACT, BF16, WD, GS>(pv[k], gv[k], m_old, v_old, h, gscale, dbc1, dbc2, m, v, pn[k]);
                mf[c * 8 + k] = m;
                vf[c * 8 + k] = v;
                lm = fmaxf(lm, __builtin_fabsf(m));
                lv = fmaxf(lv, __builtin_fabsf(v));
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

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB>
__device__ __forceinline__ void tail_block(const DevTensor &t, uint32_t lb, uint32_t n, uint32_t lane,
                                        const EriAdam8Hyper &h, float gscale, const BlockDiv &dbc1,
                                        const BlockDiv &dbc2, const Lds &L) {
    const size_t e0 = (size_t)lb * kBlock;
    ERI_GLOBAL uint8_t *mc = as_global(t.m);
    ERI_GLOBAL uint8_t *vc = as_global(t.v);
    const float a_m = as_global(t.absmax_m)[lb];
    const float a_v = as_global(t.absmax_v)[lb];
    float lm = 0.0f, lv = 0.0f;
    for (uint32_t i = lane; i < n; i += kWave) {
        const size_t e = e0 + i;
        float m, v, pn;
        adam_elem<MODE, EXACT, BF16, WD, GS>(load1<BF16>(t.p, e), load1<BF16>(t.g, e), L.map_s[mc[e]] * a_m,
                                             L.map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn);
        lm = fmaxf(lm, __builtin_fabsf(m));
        lv = fmaxf(lv, __builtin_fabsf(v));
    }
    float nam = lm, nav = lv;
    wave_max2(nam, nav);
    constexpr float ks = KEYTAB ? kKeyScale : 1.0f, ksi = KEYTAB ? kKeyScaleInv : 1.0f;
    const BlockDiv dm(nam, ks, ksi), dv(nav, ks, ksi);
    for (uint32_t i = lane; i < n; i += kWave) {
        const size_t e = e0 + i;
        float m, v, pn;
        adam_elem<MODE, EXACT, BF16, WD, GS>(load1<BF16>(t.p, e), load1<BF16>(t.g, e), L.map_s[mc[e]] * a_m,
                                             L.map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn);
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
__device__ __forceinline__ uint32_t find_row(const DevTensor *rows, uint32_t n_rows, uint32_t from, uint32_t blk) {
    uint32_t lo = from, hi = n_rows; // rows[lo].full_start <= blk
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (rows[mid].full_start <= blk) lo = mid; else hi = mid;
    }
    return lo;
}

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

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB>
__global__ __launch_bounds__(1024) void adam8_step_kernel(const DevTensor *__restrict__ rows, uint32_t n_rows,
                                                          uint32_t total_blocks, EriAdam8Hyper h,
                                                          const uint4 *__restrict__ lds_image,
                                                          const float *__restrict__ dev_scale, uint32_t chunks) {
    ERI_LDS_IMAGE;
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

    // partial last blocks first: one per row at most, handed out from the last wave backwards -- the
    // waves at the end of each range are the ones that get one full block fewer when the blocks do not
    // divide evenly, so the slower element-wise tail lands where there is slack
    for (uint32_t r = stride - 1 - wave; r < n_rows; r += stride) {
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        if (n != 0) {
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            tail_block<BF16, MODE, EXACT, WD, GS, KEYTAB>(t, (uint32_t)(t.numel / kBlock), n, lane, h, gscale, dbc1, dbc2, L);
        }
    }
    uint32_t ti = 0; // rows[ti].full_start <= blk; blk only grows, so the search restarts from ti
    const BlockWalk walk(total_blocks, chunks);
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        ti = find_row(rows, n_rows, ti, blk);
        const DevTensor t = rows[ti];
        const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
        full_block<BF16, MODE, EXACT, WD, GS, KEYTAB>(t, blk - t.full_start, lane, h, gscale, dbc1, dbc2, L);
    }
}

// ------------------------------------------------------------------------------------------
// software-pipelined step kernel for bf16 tensors
//
// Same arithmetic as adam8_step_kernel, but a wave issues the loads of its NEXT block after the
// update half of the current block (when the raw words of the current block are dead) and before
// the requantisation half, so it always has 48 bytes per lane in flight while it computes.  The
// registers of the raw words are the ones just freed, so the pipeline costs no copies; it needs
// 48 (raw) + 64 (moments) + temporaries at its peak, hence three waves per SIMD (768 threads).
// ------------------------------------------------------------------------------------------

struct RawBlock {
    u32x4 p[4], g[4];
    u32x2 m[4], v[4];
    float a_m, a_v;
    __device__ __forceinline__ void issue(const DevTensor &t, uint32_t lb, uint32_t lane) {
        const size_t e0 = (size_t)lb * kBlock;
        ERI_GLOBAL const u32x4 *pp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(t.p) + e0));
        ERI_GLOBAL const u32x4 *gp = as_global(reinterpret_cast<const u32x4 *>(static_cast<const uint16_t *>(t.g) + e0));
        ERI_GLOBAL const u32x2 *mp = as_global(reinterpret_cast<const u32x2 *>(t.m + e0));
        ERI_GLOBAL const u32x2 *vp = as_global(reinterpret_cast<const u32x2 *>(t.v + e0));
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            p[c] = __builtin_nontemporal_load(&pp[c * 64 + lane]); // each byte is touched once per step
            g[c] = __builtin_nontemporal_load(&gp[c * 64 + lane]);
            m[c] = __builtin_nontemporal_load(&mp[c * 64 + lane]);
            v[c] = __builtin_nontemporal_load(&vp[c * 64 + lane]);
        }
        a_m = as_global(t.absmax_m)[lb];
        a_v = as_global(t.absmax_v)[lb];
    }
};

template <int MODE, bool EXACT, bool WD, bool GS, int V = 0>
__global__ __launch_bounds__(768) void adam8_step_pipelined_kernel(const DevTensor *__restrict__ rows,
                                                                   uint32_t n_rows, uint32_t total_blocks,
                                                                   EriAdam8Hyper h,
                                                                   const uint4 *__restrict__ lds_image,
                                                                   const float *__restrict__ dev_scale,
                                                                   uint32_t chunks) {
    ERI_LDS_IMAGE;
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

    const uint32_t wave = __builtin_amdgcn_readfirstlane(blockIdx.x * waves_per_wg + threadIdx.x / kWave);
    // partial last blocks first: one per row at most, handed out from the last wave backwards -- the
    // waves at the end of each range are the ones that get one full block fewer when the blocks do not
    // divide evenly, so the slower element-wise tail lands where there is slack
    for (uint32_t r = stride - 1 - wave; r < n_rows; r += stride) {
        const DevTensor t = rows[r];
        const uint32_t n = (uint32_t)(t.numel % kBlock);
        if (n != 0) {
            const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
            tail_block<true, MODE, EXACT, WD, GS, true>(t, (uint32_t)(t.numel / kBlock), n, lane, h, gscale, dbc1, dbc2, L);
        }
    }
    const BlockWalk walk(total_blocks, chunks);
    uint32_t blk = walk.first;
    if (blk >= walk.end) return;

    uint32_t ti = find_row(rows, n_rows, 0, blk);
    DevTensor t = rows[ti];
    RawBlock raw;
    raw.issue(t, blk - t.full_start, lane);
    while (true) {
        // the block after this one; past the end the wave re-reads its last block (the loads must
        // stay unconditional so that the raw registers have a single definition in the loop)
        const uint32_t nblk = blk + walk.stride;
        const bool more = nblk < walk.end;
        const uint32_t pblk = more ? nblk : blk;
        const uint32_t nti = find_row(rows, n_rows, ti, pblk);
        const DevTensor nt = rows[nti];

        const uint32_t lb = blk - t.full_start;
        const float gscale = GS ? (h.grad_scale * t.grad_scale) * tscale : 1.0f;
        const size_t e0 = (size_t)lb * kBlock;
        char *p = static_cast<char *>(t.p) + e0 * 2;
        uint8_t *mc = t.m + e0;
        uint8_t *vc = t.v + e0;
        float mf[32], vf[32];
        u32x4 pw[4]; // updated parameters, packed, stored after the next block's loads are out
        float lm = 0.0f, lv = 0.0f;
        const float a_m = raw.a_m, a_v = raw.a_v;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            Raw8<true> pr, gr;
            pr.w = raw.p[c];
            gr.w = raw.g[c];
            float pv[8], gv[8], pn[8];
            pr.unpack(pv);
            gr.unpack(gv);
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                const float m_old = lds_float_at(L.map_s, code_offset(raw.m[c], k)) * a_m;
                const float v_old = lds_float_at(L.map_u, code_offset(raw.v[c], k)) * a_v;
                float m, v;
                adam_elem<MODE, EXACT, true, WD, GS>(pv[k], gv[k], m_old, v_old, h, gscale, dbc1, dbc2, m, v, pn[k]);
                mf[c * 8 + k] = m;
                vf[c * 8 + k] = v;
                lm = fmaxf(lm, __builtin_fabsf(m));
                lv = fmaxf(lv, __builtin_fabsf(v));
            }
            pw[c].x = bf16_pair(pn[0], pn[1]);
            pw[c].y = bf16_pair(pn[2], pn[3]);
            pw[c].z = bf16_pair(pn[4], pn[5]);
            pw[c].w = bf16_pair(pn[6], pn[7]);
            if (V == 1) __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
        }
        float nam = lm, nav = lv;
        wave_max2(nam, nav);
        if (lane == 0) {
            as_global(t.absmax_m)[lb] = nam;
            as_global(t.absmax_v)[lb] = nav;
        }
        raw.issue(nt, pblk - nt.full_start, lane); // prefetch: in flight during the requantisation
        if (V == 0 || V == 3) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
                __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
        }
        const BlockDiv dm(nam, kKeyScale, kKeyScaleInv), dv(nav, kKeyScale, kKeyScaleInv);
        if (dm.fast && dv.fast) {
            u32x2 mws[4], vws[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t o = c * 512 + lane * 8;
                requant8<true, true>(mf + c * 8, vf + c * 8, dm, dv, L, mws[c], vws[c]);
                if (V != 3) {
                    __builtin_nontemporal_store(mws[c], as_global(reinterpret_cast<u32x2 *>(mc + o)));
                    __builtin_nontemporal_store(vws[c], as_global(reinterpret_cast<u32x2 *>(vc + o)));
                }
            }
            if (V == 3) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const uint32_t o = c * 512 + lane * 8;
                    __builtin_nontemporal_store(mws[c], as_global(reinterpret_cast<u32x2 *>(mc + o)));
                    __builtin_nontemporal_store(vws[c], as_global(reinterpret_cast<u32x2 *>(vc + o)));
                }
            }
            if (V == 2) {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
            }
        } else {
            if (V == 2) {
#pragma unroll
                for (int c = 0; c < 4; ++c)
                    __builtin_nontemporal_store(pw[c], as_global(reinterpret_cast<u32x4 *>(p) + c * 64 + lane));
            }
            for (int c = 0; c < 4; ++c) {
                const uint32_t o = c * 512 + lane * 8;
                u32x2 mw, vw;
                requant8<false, true>(mf + c * 8, vf + c * 8, dm, dv, L, mw, vw);
                __builtin_nontemporal_store(mw, as_global(reinterpret_cast<u32x2 *>(mc + o)));
                __builtin_nontemporal_store(vw, as_global(reinterpret_cast<u32x2 *>(vc + o)));
            }
        }
        if (!more) break;
        blk = nblk;
        ti = nti;
        t = nt;
    }
}

int g_norm_waves = 4;      // waves per workgroup of the gradient-norm pass (eri_adam8_set_tuning key 4)
int g_pipelined_waves = 0; // measurement switch: waves per workgroup of the pipelined kernel (0 = 12)
int g_chunks = 8; // contiguous ranges of the block list (BlockWalk); 8 = one per accelerator die
/* The chunked walk needs the same number of workgroups in every chunk. */
static uint32_t chunks_for(uint32_t grid) {
    return (g_chunks > 1 && grid % (uint32_t)g_chunks == 0) ? (uint32_t)g_chunks : 1u;
}
int g_kernel_variant = 0; // A/B switch for measurements (eri_adam8_set_tuning); 0 is the shipped schedule

template <int MODE, bool EXACT, bool WD, bool GS>
static int launch_pipelined(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                            const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    auto k = adam8_step_pipelined_kernel<MODE, EXACT, WD, GS>;
    if (MODE == ERI_ADAM8_MODE_ERI && !EXACT && WD && !GS) { // the benchmark configuration carries the variants
        if (g_kernel_variant == 1) k = adam8_step_pipelined_kernel<MODE, EXACT, WD, GS, 1>;
        if (g_kernel_variant == 2) k = adam8_step_pipelined_kernel<MODE, EXACT, WD, GS, 2>;
        if (g_kernel_variant == 3) k = adam8_step_pipelined_kernel<MODE, EXACT, WD, GS, 3>;
    }
    if (wg > 768) wg = 768;
    if (g_pipelined_waves >= 1 && g_pipelined_waves <= 12) wg = (uint32_t)g_pipelined_waves * kWave;
    hipLaunchKernelGGL(k, dim3(grid), dim3(wg), 0, s, rows, n_rows, total_blocks, h,
                       static_cast<const uint4 *>(lds_image), dev_scale, chunks_for(grid));
    return (int)hipGetLastError();
}

template <bool BF16, int MODE, bool EXACT, bool WD, bool GS, bool KEYTAB>
static int launch_one(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                      const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    auto k = adam8_step_kernel<BF16, MODE, EXACT, WD, GS, KEYTAB>;
    hipLaunchKernelGGL(k, dim3(grid), dim3(wg), 0, s, rows, n_rows, total_blocks, h,
                       static_cast<const uint4 *>(lds_image), dev_scale, chunks_for(grid));
    return (int)hipGetLastError();
}

template <bool BF16, int MODE, bool EXACT>
static int launch_flags(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, const EriAdam8Hyper &h,
                        const void *img, const float *dev_scale, uint32_t grid, uint32_t wg, hipStream_t s) {
    const bool wd = h.weight_decay > 0.0f;
    const bool gs = (h.flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
    const bool bs = (h.flags & ERI_ADAM8_FLAG_BSEARCH) != 0;
#define ERI_GO(W, G, K) return launch_one<BF16, MODE, EXACT, W, G, K>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s)
    if (bs) { // cross-check path: only the two decay variants are built for it
        if (wd) { if (gs) ERI_GO(true, true, false); ERI_GO(true, false, false); }
        if (gs) ERI_GO(false, true, false);
        ERI_GO(false, false, false);
    }
    if (BF16 && (h.flags & ERI_ADAM8_FLAG_NO_PIPELINE) == 0) {
        if (wd) {
            if (gs) return launch_pipelined<MODE, EXACT, true, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
            return launch_pipelined<MODE, EXACT, true, false>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
        }
        if (gs) return launch_pipelined<MODE, EXACT, false, true>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
        return launch_pipelined<MODE, EXACT, false, false>(rows, n_rows, total_blocks, h, img, dev_scale, grid, wg, s);
    }
    if (wd) { if (gs) ERI_GO(true, true, true); ERI_GO(true, false, true); }
    if (gs) ERI_GO(false, true, true);
    ERI_GO(false, false, true);
#undef ERI_GO
}

int launch_step(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag,
                const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, uint32_t grid, uint32_t wg,
                void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool exact = (h.flags & ERI_ADAM8_FLAG_EXACT_PARAM) != 0;
    if (h.mode == ERI_ADAM8_MODE_BNB) { // plain kernel, slot table, IEEE arithmetic; the decay is a factor
        const bool wd = h.weight_decay != 1.0f;
        const bool gs = (h.flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
#define ERI_BNB(B, W, G) return launch_one<B, ERI_ADAM8_MODE_BNB, true, W, G, true>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s)
        if (dtype_tag == ERI_DTYPE_F32) {
            if (wd) { if (gs) ERI_BNB(false, true, true); ERI_BNB(false, true, false); }
            if (gs) ERI_BNB(false, false, true);
            ERI_BNB(false, false, false);
        }
        if (wd) { if (gs) ERI_BNB(true, true, true); ERI_BNB(true, true, false); }
        if (gs) ERI_BNB(true, false, true);
        ERI_BNB(true, false, false);
#undef ERI_BNB
    }
    if (dtype_tag == ERI_DTYPE_F32) {
        if (h.mode == ERI_ADAM8_MODE_L2)
            return launch_flags<false, ERI_ADAM8_MODE_L2, true>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
        return launch_flags<false, ERI_ADAM8_MODE_ERI, true>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
    }
    if (h.mode == ERI_ADAM8_MODE_L2) {
        if (exact) return launch_flags<true, ERI_ADAM8_MODE_L2, true>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
        return launch_flags<true, ERI_ADAM8_MODE_L2, false>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
    }
    if (exact) return launch_flags<true, ERI_ADAM8_MODE_ERI, true>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
    return launch_flags<true, ERI_ADAM8_MODE_ERI, false>(rows, n_rows, total_blocks, h, lds_image, dev_scale, grid, wg, s);
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
        uint32_t ti = find_row(rows, n_rows, 0, walk.first);
        Raw8<BF16> raw[4];
        {
            const DevTensor t = rows[ti];
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
                ti = find_row(rows, n_rows, ti, nblk);
                const DevTensor t = rows[ti];
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

int launch_grad_sumsq(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag, double *partial,
                      uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype_tag == ERI_DTYPE_F32)
        hipLaunchKernelGGL(grad_sumsq_kernel<false>, dim3(grid), dim3(g_norm_waves * kWave), 0, s, rows, n_rows, total_blocks, partial, chunks_for(grid));
    else
        hipLaunchKernelGGL(grad_sumsq_kernel<true>, dim3(grid), dim3(g_norm_waves * kWave), 0, s, rows, n_rows, total_blocks, partial, chunks_for(grid));
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
                                                          uint32_t total_blocks, EriAdam8Hyper h,
                                                          const float *__restrict__ lds_image,
                                                          const float *__restrict__ dev_scale,
                                                          double *__restrict__ err /* [2 * n_rows] */) {
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
            adam_elem<MODE, true, BF16, WD, GS>(load1<BF16>(t.p, e), load1<BF16>(t.g, e), map_s[mc[e]] * a_m,
                                                map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn);
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
            adam_elem<MODE, true, BF16, WD, GS>(load1<BF16>(t.p, e), load1<BF16>(t.g, e), map_s[mc[e]] * a_m,
                                                map_u[vc[e]] * a_v, h, gscale, dbc1, dbc2, m, v, pn);
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

int launch_quant_error(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag,
                       const EriAdam8Hyper &h, const void *lds_image, const float *dev_scale, double *err,
                       uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const float *img = static_cast<const float *>(lds_image);
    hipLaunchKernelGGL(zero_f64_kernel, dim3(64), dim3(256), 0, s, err, 2 * n_rows);
    const bool bf16 = dtype_tag != ERI_DTYPE_F32, l2 = h.mode == ERI_ADAM8_MODE_L2;
    const bool wd = h.weight_decay > 0.0f, gs = (h.flags & ERI_ADAM8_FLAG_GRAD_SCALE) != 0;
#define ERI_QE(B, M, W, G) hipLaunchKernelGGL((quant_error_kernel<B, M, W, G>), dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, h, img, dev_scale, err)
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

__device__ __forceinline__ uint32_t find_elem_row(const ElemRow *rows, uint32_t n_rows, uint32_t from, uint32_t blk) {
    uint32_t lo = from, hi = n_rows;
    while (hi - lo > 1) {
        const uint32_t mid = (lo + hi) >> 1;
        if (rows[mid].full_start <= blk) lo = mid; else hi = mid;
    }
    return lo;
}

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
template <bool BF16, bool MASTER>
__device__ __forceinline__ void adamw32_block(const ElemRow &t, size_t e0, uint32_t lane, const EriAdamW32Hyper &h,
                                              float omb1, float omb2, float neg_lr) {
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
        for (int k = 0; k < 8; ++k) adamw32_elem(pv[k], gv[k], mv[k], vv[k], h, omb1, omb2, neg_lr, pn[k]);
        store8<BF16>(p, o, pn);
        if (MASTER) store8<false>(w, o, pn);
        store8<false>(m, o, mv);
        store8<false>(v, o, vv);
    }
}

template <bool BF16>
__global__ __launch_bounds__(256) void adamw32_kernel(const ElemRow *__restrict__ rows, uint32_t n_rows,
                                                      uint32_t total_blocks, EriAdamW32Hyper h, uint32_t chunks) {
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
        for (uint32_t i = lane; i < n; i += kWave) {
            float m = mp[e0 + i], v = vp[e0 + i], pn;
            const float pf = wp ? wp[e0 + i] : load1<BF16>(t.a, e0 + i);
            adamw32_elem(pf, load1<BF16>(t.b, e0 + i), m, v, h, omb1, omb2, neg_lr, pn);
            mp[e0 + i] = m;
            vp[e0 + i] = v;
            if (wp) wp[e0 + i] = pn;
            store1<BF16>(t.a, e0 + i, pn);
        }
    }
    uint32_t ti = 0;
    const BlockWalk walk(total_blocks, chunks);
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        ti = find_elem_row(rows, n_rows, ti, blk);
        const ElemRow t = rows[ti];
        const size_t e0 = (size_t)(blk - t.full_start) * kBlock;
        if (t.e) adamw32_block<BF16, true>(t, e0, lane, h, omb1, omb2, neg_lr);
        else adamw32_block<BF16, false>(t, e0, lane, h, omb1, omb2, neg_lr);
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
    uint32_t ti = 0;
    const BlockWalk walk(total_blocks, chunks);
    for (uint32_t blk = walk.first; blk < walk.end; blk += walk.stride) {
        ti = find_elem_row(rows, n_rows, ti, blk);
        const ElemRow t = rows[ti];
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
                   const EriAdamW32Hyper &h, uint32_t grid, void *stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (dtype_tag == ERI_DTYPE_F32)
        hipLaunchKernelGGL(adamw32_kernel<false>, dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, h, chunks_for(grid));
    else
        hipLaunchKernelGGL(adamw32_kernel<true>, dim3(grid), dim3(256), 0, s, rows, n_rows, total_blocks, h, chunks_for(grid));
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
