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

/* One tensor as the kernels see it (64 bytes, read through scalar loads). */
struct DevTensor {
    void *p;
    const void *g;
    uint8_t *m;
    uint8_t *v;
    float *absmax_m;
    float *absmax_v;
    uint64_t numel;
    uint32_t block_start; /* first block of this tensor within its dtype group */
    float grad_scale;
};
static_assert(sizeof(DevTensor) == 64, "DevTensor must stay 64 bytes");

/*
 * Requantisation without a search.  For x in [-1, 1] the top bits of |x| (sign, exponent and the
 * leading kMant mantissa bits) select a slot; the slots are narrow enough that at most one
 * midpoint of the map lies inside any of them, so
 *     code(x) = slot.lo + (x > slot.mid)
 * equals the number of midpoints below x, i.e. the binary search's answer, ties included.
 * Slot 0 also takes everything smaller than 2^(kExp0-127); the last slot of each sign takes NaN
 * and returns code 0, which is what a search does with NaN (every comparison false).
 */
struct KeySlot {
    float mid;   /* the one midpoint inside the slot, +inf if there is none */
    uint32_t lo; /* number of midpoints below every value of the slot */
};

constexpr uint32_t kKeyExp0 = 106; /* biased exponent of the first binade that gets its own slots */
constexpr uint32_t kSMant = 6;     /* signed map: 64 slots per binade */
constexpr uint32_t kUMant = 7;     /* unsigned map: 128 slots per binade */
constexpr uint32_t kSShift = 23 - kSMant;
constexpr uint32_t kUShift = 23 - kUMant;
constexpr uint32_t kSBase = kKeyExp0 << kSMant;
constexpr uint32_t kUBase = kKeyExp0 << kUMant;
constexpr uint32_t kSSlots = ((127 - kKeyExp0) << kSMant) + 1; /* through x == 1.0 */
constexpr uint32_t kUSlots = ((127 - kKeyExp0) << kUMant) + 1;
constexpr uint32_t kSPerSign = kSSlots + 1; /* + the NaN slot */
constexpr uint32_t kUCount = kUSlots + 1;

/* Byte offsets inside the LDS image. */
constexpr uint32_t kOffMapS = 0;                              /* 256 floats: code -> value */
constexpr uint32_t kOffMapU = kOffMapS + 1024;                /* 256 floats */
constexpr uint32_t kOffMidS = kOffMapU + 1024;                /* 255 midpoints + one +inf */
constexpr uint32_t kOffMidU = kOffMidS + 1024;
constexpr uint32_t kOffKeyS = kOffMidU + 1024;                /* 2 * kSPerSign slots: positive, negative */
constexpr uint32_t kOffKeyU = kOffKeyS + 2 * kSPerSign * 8;   /* kUCount slots */
constexpr uint32_t kLdsImageBytesRaw = kOffKeyU + kUCount * 8;
constexpr uint32_t kLdsImageBytes = (kLdsImageBytesRaw + 15u) & ~15u;

/* Launchers implemented in eri_adam8_kernels.hip; `stream` is a hipStream_t.  All return a
 * hipError_t as int.  `lds_image` is the device copy of the kLdsImageBytes table image. */
int launch_step(const DevTensor *rows, uint32_t n_rows, uint32_t total_blocks, int dtype_tag,
                const EriAdam8Hyper &h, const void *lds_image, uint32_t grid, uint32_t wg, void *stream);
int launch_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel, void *stream);
int launch_dequantize(const uint8_t *codes, const float *absmax, int signed_map, uint64_t numel, float *out,
                      const void *lds_image, void *stream);
int launch_quantize(const float *x, int signed_map, uint64_t numel, uint8_t *codes, float *absmax,
                    const void *lds_image, void *stream);

} // namespace eri
#endif
