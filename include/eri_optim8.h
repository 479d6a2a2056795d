/*
 * eri_optim8 -- C ABI of the MI355X (gfx950) blockwise 8-bit AdamW step for EriDiffusion.
 *
 * Everything EriDiffusion's optimizer path needs from native code crosses this header: device
 * storage (hipMalloc / hipMemcpyAsync, no CUDA shim), the multi-tensor launch table, and the
 * single-pass step kernel.  Plain pointers and sizes only; a Rust `extern "C"` block, ctypes or
 * cgo can bind it as it stands.
 *
 * Conventions, taken from the reference's own Rust<->C seam:
 *   - every call returns int: 0 on success, a positive hipError_t from the runtime, or a negative
 *     EriStatus for argument errors.  The reference's launchers return 0 or the raw cudaError_t
 *     (crates/core/cuda/narrow_strided.cu:93-97) and its Rust side turns non-zero into
 *     Err(TensorOp("... failed with code N")) (crates/core/src/tensor_narrow.rs:221-227).
 *   - streams are passed as void* and NULL means the default stream
 *     (crates/core/src/device.rs:69-71, tensor_narrow.rs:197-201).
 *   - dtype tags are F32=0, F16=1, BF16=2, I32=3 (crates/core/src/cuda/dtype_tag.rs:3-19);
 *     the optimizer accepts F32 and BF16 parameters, with gradients of the same dtype or F32.
 *   - nothing here synchronises the device unless its name says so; the step is stream-ordered.
 *   - the library never takes ownership of parameter, gradient or state memory.
 */
#ifndef ERI_OPTIM8_H
#define ERI_OPTIM8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ERI_ADAM8_BLOCK 2048u /* elements per quantisation block */

typedef enum EriDTypeTag { ERI_DTYPE_F32 = 0, ERI_DTYPE_F16 = 1, ERI_DTYPE_BF16 = 2, ERI_DTYPE_I32 = 3 } EriDTypeTag;

typedef enum EriStatus {
    ERI_OK = 0,
    ERI_ERR_NULL = -1,        /* a required pointer is NULL */
    ERI_ERR_ALIGN = -2,       /* p/g/m/v not 16-byte aligned, absmax not 4-byte aligned */
    ERI_ERR_EMPTY = -3,       /* numel == 0 ("Empty tensor for quantization", adam8bit_enhanced.rs:46-50) */
    ERI_ERR_DTYPE = -4,       /* dtype tag other than F32 / BF16 */
    ERI_ERR_BLOCK_START = -5, /* block_start is not the running sum of ceil(numel / 2048) */
    ERI_ERR_ARG = -6,         /* any other bad argument (mode, count, size, kind) */
    ERI_ERR_TOO_LARGE = -7,   /* more than 2^31 - 1 blocks in one table */
    ERI_ERR_INTERNAL = -8     /* the lookup tables failed their self-check, or pinned staging memory is unavailable */
} EriStatus;

/* Message for the last failing call on this thread ("" if none).  Never NULL. */
const char *eri_last_error(void);
/* Lets a layer built on this ABI (include/eri_adam8bit.h, a language binding) leave its own message. */
void eri_set_last_error(const char *message);

/* ---------------------------------------------------------------------------------------------
 * Device storage.  Replaces the cudarc-backed seam of the reference:
 *   cuda_malloc_zeroed(dev, size) -> *mut u8          crates/core/src/cuda/mod.rs:47-66
 *   MemoryPool::allocate_raw_memory                    crates/core/src/memory.rs:289-311
 *   cuda_alloc_pinned_host / cuda_free_pinned_host /
 *   cuda_memcpy_async(dst, src, bytes, kind, stream)   crates/core/cuda/utils_pinned.cu:4-20
 * `kind` keeps the reference's encoding: 1 = host->device, 2 = device->host, 3 = device->device,
 * anything else = let the runtime infer it.
 * ------------------------------------------------------------------------------------------- */
int eri_hip_device_count(int *count);
int eri_hip_set_device(int device);
int eri_hip_get_device(int *device);
/* 256-byte aligned, zero-filled.  Allocations of 64 MB and more are allocated, released and allocated
 * again before they are handed out: on MI355X the first physical placement a large request receives
 * sustains visibly less bandwidth than the one it receives after the range went back to the driver.
 * Environment: ERI_HIP_MALLOC_RECYCLE=0 switches that off. */
int eri_hip_malloc_zeroed(int device, size_t bytes, void **out);
int eri_hip_free(void *ptr);
void *eri_hip_host_alloc(size_t bytes);                          /* pinned; NULL on failure */
int eri_hip_host_free(void *ptr);
int eri_hip_memcpy_async(void *dst, const void *src, size_t bytes, int kind, void *stream);
/* Byte fill through the runtime's own memset.  Not for a stream that is being captured into a HIP graph:
 * the optimizer calls below clear what they need with a small kernel of their own and stay capturable. */
int eri_hip_memset_async(void *dst, int value, size_t bytes, void *stream);
int eri_hip_stream_create(void **stream);                        /* default priority */
int eri_hip_stream_sync(void *stream);
int eri_hip_stream_destroy(void *stream);
int eri_hip_mem_info(size_t *free_bytes, size_t *total_bytes);
/* What the runtime knows about an address: memory it never allocated (malloc, the stack, a mapped file) is
 * ERI_PTR_UNKNOWN, and a kernel that touches it faults the device.  The calls that take device pointers from
 * code which is usually holding host buffers at that moment (eri_adam8_quantize / _dequantize and the
 * optimizer calls built on them) ask this first and refuse with ERI_ERR_ARG; the step's own calls do not (their
 * tables hold thousands of pointers and are rebuilt on a trainer's hot path). */
enum { ERI_PTR_UNKNOWN = 0, ERI_PTR_PINNED_HOST = 1, ERI_PTR_DEVICE = 2, ERI_PTR_MANAGED = 3 };
int eri_hip_pointer_kind(const void *p, int *kind);

/* A device memory pool with lanes: ONE device allocation cut into `lanes` equal parts, each handing out
 * 256-byte aligned, zero-filled pieces from its start upwards.  It exists for placement.  On MI355X a kernel
 * that reads and writes several arrays at once (the optimizer step: parameters, gradients, two state arrays)
 * runs 10-17 % faster when the 8-bit states lie 32 GiB or more away from the parameters and gradients in
 * device memory than with everything adjacent, and separate hipMalloc calls give no say over that; inside
 * one allocation distances are what the caller makes them.  Meant as the backing store of the reference's
 * MemoryPool (crates/core/src/memory.rs:243-311 allocates one block per request through cuda_malloc_zeroed):
 * a lane per kind of tensor -- the reference already keeps one pool per dtype, so U8 states and BF16 parameters
 * fall into different lanes by themselves.
 * bytes = 0 takes nine tenths of the free device memory; lanes = 0 makes as many lanes of exactly 48 GiB as fit
 * into `bytes` (a smaller pool is a single lane).
 * eri_hip_pool_release gives one piece back: the top piece of a lane lowers the lane's fill level, any other is
 * kept and handed out again to the next request of exactly its size in that lane (optimizer states that are
 * replaced, e.g. by loading a checkpoint, have the size of the ones they replace).  eri_hip_pool_reset empties
 * every lane.  eri_hip_pool_destroy ends the creator's use of the pool: nothing more is handed out, and the
 * allocation is freed at once unless somebody else holds the pool through eri_hip_pool_retain (the optimizers do,
 * once per state they took from it, so that a state destroyed after the pool still has somewhere to give its
 * piece back to); then it is freed when the last of them lets go with eri_hip_pool_unretain.  Calls on one pool
 * may come from several threads. */
typedef struct EriHipPool EriHipPool;
int eri_hip_pool_create(int device, size_t bytes, uint32_t lanes, EriHipPool **out);
/* lane counts modulo the pool's lanes.  The piece is cleared by the runtime's synchronous memset: it is zero,
 * for work on any stream, when the call returns. */
int eri_hip_pool_alloc_zeroed(EriHipPool *pool, uint32_t lane, size_t bytes, void **out);
/* The same, cleared by a small kernel on `stream` instead: the host does not wait, the call may sit inside a
 * stream capture, and the piece is zero for whatever follows it on that stream (work on another stream has to be
 * ordered after it by the caller). */
int eri_hip_pool_alloc_zeroed_async(EriHipPool *pool, uint32_t lane, size_t bytes, void *stream, void **out);
/* Gives back a piece with the byte count it was requested with.  The caller orders the release after the last
 * use of the piece (the next owner clears it on its own stream or through the synchronous memset). */
int eri_hip_pool_release(EriHipPool *pool, void *ptr, size_t bytes);
int eri_hip_pool_info(const EriHipPool *pool, uint32_t *lanes, size_t *lane_bytes);
int eri_hip_pool_lane_used(const EriHipPool *pool, uint32_t lane, size_t *used_bytes);
int eri_hip_pool_reset(EriHipPool *pool);
int eri_hip_pool_destroy(EriHipPool *pool);
int eri_hip_pool_retain(EriHipPool *pool);
int eri_hip_pool_unretain(EriHipPool *pool);

/* ---------------------------------------------------------------------------------------------
 * The optimizer step.
 * ------------------------------------------------------------------------------------------- */

/* Which reference function the arithmetic follows. */
typedef enum EriAdam8Mode {
    ERI_ADAM8_MODE_ERI = 0, /* Adam8bit::step,   src/trainers/adam8bit_enhanced.rs:202-291:
                               p -= step_size * (m / (sqrt(v) + eps) + wd * p) */
    ERI_ADAM8_MODE_L2 = 1,  /* Adam8bit::update, src/trainers/adam8bit.rs:101-208:
                               g += wd * p; p -= cast(lr * (m/bc1) / (sqrt(max(v/bc2, 0)) + eps)) */
    ERI_ADAM8_MODE_BNB = 2  /* not in the reference; the update of the library the state format comes from
                               (bitsandbytes 8-bit blockwise Adam): p = (p - step_size * m / (sqrt(v) +
                               eps*sqrt(bc2))) * (1 - lr*wd), and a first-moment code whose map value has the
                               other sign than the moment moves one entry toward the moment's sign.  With
                               wd = 0 this is the textbook Adam formula.  Moments as in ERI.  Not
                               available to eri_adam8_quant_error. */
} EriAdam8Mode;

enum {
    ERI_ADAM8_FLAG_GRAD_SCALE = 1u << 0,  /* multiply gradients by hyper.grad_scale * tensor.grad_scale */
    ERI_ADAM8_FLAG_EXACT_PARAM = 1u << 1, /* BF16 parameters come out with the bits of the chain of individually
                                             rounded IEEE operations (F32 parameters always do): every element
                                             whose rounding the faster arithmetic cannot vouch for is recomputed
                                             with IEEE sqrt and divide.  Without the flag BF16 parameters are
                                             within one BF16 unit in the last place of those bits */
    ERI_ADAM8_FLAG_BSEARCH = 1u << 2,     /* requantise by binary search of the LDS midpoint table
                                             instead of the float-keyed slot table (same codes; runs on
                                             the plain one-wave-per-block kernel whatever the table size) */
    ERI_ADAM8_FLAG_NO_PIPELINE = 1u << 3, /* use the plain one-wave-per-block kernel: not the one that
                                             prefetches the next block (large tables), not the
                                             four-waves-per-block one (small tables).  Same results; a
                                             cross-check */
    ERI_ADAM8_FLAG_CLIP_FROM_TABLE = 1u << 4, /* also multiply gradients by the clip factor the last
                                             eri_adam8_grad_norm left in the table (device memory) */
    ERI_ADAM8_FLAG_EMA = 1u << 6,         /* after the update, every row that has an ema_shadow also gets
                                             shadow = ema_decay*shadow + (1 - ema_decay)*p', the EMA update of
                                             src/trainers/ema_enhanced.rs:91-100 on the parameter as it was just
                                             stored.  Tables of BF16 parameters (BF16 or F32 gradients) in mode
                                             ERI beyond the small-table kernel's range do it inside the step
                                             kernel (the new parameter is still in registers: the separate
                                             sweep's read of p is saved); every other table runs one EMA sweep
                                             right after the step, in the same call.  Same results either way */
    ERI_ADAM8_FLAG_ONE_WAVE = 1u << 5     /* take the kernel of the largest tables whatever the size: one
                                             wave per block with the next block's loads in flight.  Same
                                             results; lets tests reach every kernel with small inputs */
};

/* Per-step scalars, already cast where the reference casts them.  Fill with eri_adam8_hyper_pack. */
typedef struct EriAdam8Hyper {
    /* BNB: eps holds (float)(eps * sqrt(bc2)) and weight_decay the factor (float)(1 - lr*wd). */
    float beta1, beta2; /* (float)beta                               adam8bit_enhanced.rs:256,260 */
    float omb1, omb2;   /* ERI: 1.0f - (float)beta; L2: (float)(1.0 - beta)    :256,260 / adam8bit.rs:142,151 */
    float eps;          /* (float)eps                                :263 */
    float weight_decay; /* (float)wd                                 :268 */
    float step_size;    /* ERI: (float)(lr * sqrt(bc2) / bc1), f64 inside      :213-215,274; L2: (float)lr */
    float bc1, bc2;     /* L2: (float)(1 - beta^max(step,1))         adam8bit.rs:164-178 */
    float grad_scale;   /* used with ERI_ADAM8_FLAG_GRAD_SCALE       pipeline_flux_lora_sequential.rs:1198-1213 */
    int32_t mode;       /* EriAdam8Mode */
    uint32_t flags;     /* ERI_ADAM8_FLAG_* */
    float ema_decay;    /* used with ERI_ADAM8_FLAG_EMA: the effective decay of this step
                           (eri_ema_effective_decay, ema_enhanced.rs:106-127); eri_adam8_hyper_pack leaves 0 */
    uint32_t reserved;  /* 0 */
} EriAdam8Hyper;

/* `step` is the optimizer's counter after its increment for ERI (adam8bit_enhanced.rs:203) and the
 * counter as it stands when update() runs for L2 (adam8bit.rs:164; step() bumps it afterwards). */
int eri_adam8_hyper_pack(double lr, double beta1, double beta2, double eps, double weight_decay,
                         uint64_t step, int mode, uint32_t flags, EriAdam8Hyper *out);

/* One row of the launch table: a parameter tensor, its gradient and its 8-bit state.
 * m/v hold numel codes, absmax_* hold ceil(numel / 2048) floats.  All device pointers.
 * Rows are plain data: zero the struct first, so that fields added later read as "not used". */
typedef struct EriAdam8Tensor {
    void *p;              /* the updated parameters are written here */
    const void *g;        /* gradients: the dtype of p, or F32 if grad_f32 is set */
    uint8_t *m;           /* first-moment codes (signed dynamic map) */
    uint8_t *v;           /* second-moment codes (unsigned dynamic map) */
    float *absmax_m;      /* per-block scale of m */
    float *absmax_v;      /* per-block scale of v */
    uint64_t numel;
    uint64_t block_start; /* index of this tensor's first block = sum of the blocks before it */
    int32_t dtype_tag;    /* ERI_DTYPE_F32 or ERI_DTYPE_BF16: the dtype of p */
    float grad_scale;     /* per-layer multiplier (pipeline_flux_lora_sequential.rs:759-766);
                             read only with ERI_ADAM8_FLAG_GRAD_SCALE */
    const void *p_src;    /* NULL: p is updated in place (Parameter::apply_update, adam8bit_enhanced.rs:275).
                             Otherwise the old parameters are read from p_src (dtype of p, numel elements,
                             not overlapping p unless equal to it) and the new ones written to p, which is
                             Adam8bit::update(name, param, grad) -> new tensor (adam8bit.rs:101-208) without a copy */
    int32_t grad_f32;     /* non-zero with BF16 parameters: g holds F32 elements, which enter the arithmetic
                             unrounded -- the reference casts every gradient to F32 and never rounds it
                             (adam8bit_enhanced.rs:231-235, adam8bit.rs:110).  Such rows form a group of their
                             own with its own launch; the same three kernels serve it (by table size).
                             Must be 0 for F32 parameters */
    int32_t reserved;     /* 0 */
    void *ema_shadow;     /* NULL, or the EMA shadow of this parameter (dtype of p, numel elements, 16-byte aligned):
                             updated by steps that carry ERI_ADAM8_FLAG_EMA */
} EriAdam8Tensor;

typedef struct EriAdam8Table EriAdam8Table; /* device-resident copy of a launch table */

/* Loads the quantisation tables onto the current device.  Optional: the first table does it. */
int eri_adam8_init(void);

/* The two 256-entry maps (code -> value in [-1, 1] / [0, 1]) the states are expressed in. */
int eri_adam8_get_maps(float *signed256, float *unsigned256);

/* Codes of 0.0 (127 / 0) and absmax 0: the state of a zeros tensor (adam8bit_enhanced.rs:179-197).
 * Device pointers, as in a row of the launch table; written by a kernel on `stream`. */
int eri_adam8_state_init(uint8_t *m, uint8_t *v, float *absmax_m, float *absmax_v, uint64_t numel,
                         void *stream);

/* Validates `rows` and uploads them.  The steady-state step then allocates nothing.
 * The upload is asynchronous on `stream`.  A later call that reads the table on another stream is ordered
 * after the upload by the library (the other stream waits for the upload's event, the host does not);
 * only a stream that is being captured into a HIP graph cannot wait for an event outside the graph, and
 * there the host waits for the upload once instead. */
int eri_adam8_table_create(const EriAdam8Tensor *rows, uint32_t n, void *stream, EriAdam8Table **out);
/* Same tensors (count, numel, dtype of parameters and gradients), new pointers / grad_scale -- e.g. fresh
 * gradient buffers, or the fresh output tensors of a functional update. */
int eri_adam8_table_update(EriAdam8Table *table, const EriAdam8Tensor *rows, uint32_t n, void *stream);
int eri_adam8_table_destroy(EriAdam8Table *table);
int eri_adam8_table_info(const EriAdam8Table *table, uint64_t *total_numel, uint64_t *total_blocks);

/* One optimizer step over every tensor of the table: one kernel launch per dtype present. */
int eri_adam8_step_table(EriAdam8Table *table, const EriAdam8Hyper *hyper, void *stream);

/* Global L2 norm of every gradient of the table and the clip factor it implies, both left in device
 * memory owned by the table -- no host round trip (the reference reads one scalar back per tensor:
 * compute_gradient_norm, src/trainers/pipeline_flux_lora_sequential.rs:1939-1950).
 *   norm  = (float)sqrt(sum of g*g), squares and per-block sums in fp32, blocks added in f64
 *   scale = max_norm / (norm + denom_eps) if max_norm > 0 and norm is finite and above max_norm, else 1
 * denom_eps = 0 reproduces clip_gradients (pipeline_flux_lora_sequential.rs:1198-1213), 1e-6
 * clip_grads_global_norm_fp32_tensors (crates/training/src/optimizer.rs:58-85).  A following step with
 * ERI_ADAM8_FLAG_CLIP_FROM_TABLE applies the factor inside the kernel instead of rewriting gradients. */
int eri_adam8_grad_norm(EriAdam8Table *table, float max_norm, float denom_eps, void *stream);
/* A table of gradients only, for tensors that take part in the global norm but not in the 8-bit step (the short
 * tensors a trainer keeps in 32-bit moments, pipeline_flux_lora_1024.rs:451, are clipped by the same global
 * norm, :691-697).  Of each row only g, numel, block_start, dtype_tag and grad_f32 are read.  Such a table can
 * be updated, normed and destroyed like any other; the step and the statistics pass refuse it. */
int eri_adam8_grad_table_create(const EriAdam8Tensor *rows, uint32_t n, void *stream, EriAdam8Table **out);
/* The norm pass over the gradients of two tables as if they were one: one norm, one clip factor, left in
 * memory owned by `table` and used by both tables from then on (the reads below and
 * ERI_ADAM8_FLAG_CLIP_FROM_TABLE work on either) until one of them is normed again; `table` must outlive that
 * use.  The per-block sums are added in the order: groups of `table`, groups of `also`. */
int eri_adam8_grad_norm_joint(EriAdam8Table *table, EriAdam8Table *also, float max_norm, float denom_eps, void *stream);
/* Device address of the clip factor the table's last norm pass left (one float), for a kernel outside the
 * table that has to apply the same factor: eri_adamw32_step_multi_scaled.  Valid until the next norm pass. */
int eri_adam8_grad_norm_scale_ptr(const EriAdam8Table *table, const float **dev_scale);
/* The same pass for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses
 * that forbid hipMalloc).  It has no counterpart in the reference.  eri_adam8_grad_norm allocates the
 * per-wave partial sums and the result words on a table's first call; this variant allocates nothing:
 * the partial sums go to a static device array of the library (384 KiB per device, 24,576 per-wave
 * pairs; a table whose pass needs more is refused with ERI_ERR_TOO_LARGE -- none does on a 256-CU
 * MI355X) and the result to `result`, 16 bytes of device memory the caller owns, 8-byte aligned:
 * {float norm, float scale, uint64 count of non-finite elements}.  A following step with
 * ERI_ADAM8_FLAG_CLIP_FROM_TABLE, and the two read calls below, read `result` until the next norm pass
 * of the table: the caller keeps it allocated that long (the library holds the bare address and cannot
 * tell whether it still is).  All calls on one device share the array: two such
 * calls that overlap in time on one device (different streams, different tables) race.  Nothing in
 * the array has to start at zero (every wave of a pass writes its pair before the pair is read). */
int eri_adam8_grad_norm_static(EriAdam8Table *table, float max_norm, float denom_eps, void *result, void *stream);
/* Copies the last norm and clip factor to the host; waits for `stream`. */
int eri_adam8_grad_norm_read(EriAdam8Table *table, float *norm, float *scale, void *stream);
/* How many gradient elements of the table were NaN or +-infinity in the last eri_adam8_grad_norm; waits
 * for `stream`.  Such values propagate through the step (a NaN gradient gives a NaN parameter, as with
 * the reference's tensor ops), so a trainer can check this, or the norm, before it steps (the
 * reference's trainers test the loss instead: pipeline_flux_lora_sequential.rs:1137).
 * The count costs nothing on clean gradients: elements are examined only in blocks whose sum of
 * squares is not finite. */
int eri_adam8_grad_nonfinite_read(EriAdam8Table *table, uint64_t *count, void *stream);

/* Quantisation error the next step will incur: a read-only pass that forms the new moments exactly as
 * eri_adam8_step_table(table, hyper) would, quantises them and accumulates |value - dequantised value|.
 * eri_adam8_quant_error_read then returns the mean over tensors of the per-tensor mean absolute error
 * of the first and of the second moment -- quantization_stats(), adam8bit_enhanced.rs:318-327, whose
 * per-tensor `quantization_error` is the same mean (:93-100).  Diagnostics; costs one read pass. */
int eri_adam8_quant_error(EriAdam8Table *table, const EriAdam8Hyper *hyper, void *stream);
int eri_adam8_quant_error_read(EriAdam8Table *table, float *m_error, float *v_error, void *stream);

/* Diagnostics, no counterpart in the reference: one launch that moves the bytes of a step over the table's
 * BF16 rows (BF16 gradients) and does nothing else -- every full block read as the step kernel reads it and
 * written back unchanged, in the launch shape of the kernel that takes the largest tables.  Its duration is what
 * the device's memory system gives the step's mix of read and written streams where the caller has placed them,
 * the figure a step's duration is to be read against (`bench.py --kernel traffic`).  Partial last blocks are
 * left out.  No data changes. */
int eri_adam8_traffic_probe(EriAdam8Table *table, void *stream);

/* Convenience for callers that keep no handle: keeps one cached table per calling thread and
 * re-uploads it only when `rows` changed since that thread's last call. */
int eri_adam8_step_multi(const EriAdam8Tensor *rows, uint32_t n, const EriAdam8Hyper *hyper, void *stream);

/* Copies the host image of the kernel's lookup tables (the bytes every workgroup stages into LDS)
 * into `out` (capacity `cap`) and reports its size and the byte offsets of its six parts:
 * signed map, unsigned map, signed midpoints, unsigned midpoints, signed slots, unsigned slots.
 * No device is touched; the CPU tests replay the kernel's slot lookup against it. */
int eri_adam8_table_image(void *out, size_t cap, size_t *bytes, uint32_t offsets[6]);

/* Blockwise state <-> fp32, for checkpoints that store unquantised moments
 * (get_state_as_tensors / load_state_from_tensors, src/trainers/adam8bit.rs:296-329).
 * signed_map != 0 selects the first-moment map.  Every pointer is memory a kernel can reach (device, pinned
 * host or managed): the conversion runs on the device, on `stream`; ordinary host memory is refused. */
int eri_adam8_dequantize(const uint8_t *codes, const float *absmax, int signed_map, uint64_t numel,
                         float *out, void *stream);
int eri_adam8_quantize(const float *x, int signed_map, uint64_t numel, uint8_t *codes, float *absmax,
                       void *stream);

/* ---------------------------------------------------------------------------------------------
 * 32-bit sibling: fused multi-tensor AdamW with fp32 moments, for tensors kept out of the 8-bit
 * path.  Arithmetic of AdamW::step_with_grads (crates/common/optim/src/adamw.rs:20-58), one rounded
 * fp32 operation per line there: no bias correction, decoupled decay,
 *   m = m*b1 + g*(1-b1);  v = v*b2 + (g*g)*(1-b2);  p = p + ((m/(sqrt(v)+eps)) + p*wd) * (-lr)
 * with p cast back to its dtype.  It replaces one launch and one temporary per operation there, and
 * the never-built fused kernels of src/kernels/fused_adam.cu:108-148.
 * ------------------------------------------------------------------------------------------- */
typedef struct EriAdamW32Tensor {
    void *p;          /* F32 or BF16, updated in place */
    const void *g;    /* same dtype as p */
    float *m;         /* fp32 first moment, numel elements */
    float *v;         /* fp32 second moment */
    float *master;    /* NULL, or an fp32 master copy of p (numel elements): the step then reads and writes
                         the master and stores its rounded value in p -- mixed precision as in
                         src/kernels/fused_adam.cu:151-193, with the arithmetic above */
    uint64_t numel;
    int32_t dtype_tag;
    float grad_scale; /* per-layer multiplier of the gradients, read by eri_adamw32_step_multi_scaled only;
                         0 (a zeroed row) reads as 1 */
} EriAdamW32Tensor;

typedef struct EriAdamW32Hyper {
    float lr, beta1, beta2, eps, weight_decay; /* AdamWCfg, adamw.rs:7-8; lr is the per-call argument */
} EriAdamW32Hyper;

/* One launch per dtype over all rows; keeps a cached device copy of the rows per calling thread. */
int eri_adamw32_step_multi(const EriAdamW32Tensor *rows, uint32_t n, const EriAdamW32Hyper *hyper, void *stream);
/* The same step with every gradient first multiplied by (grad_scale * row.grad_scale) * (*dev_scale), one rounded
 * fp32 product of the gradient with that factor, the factor formed in this order -- what the 8-bit step does with
 * ERI_ADAM8_FLAG_GRAD_SCALE and ERI_ADAM8_FLAG_CLIP_FROM_TABLE, so that tensors kept in 32-bit moments are unscaled
 * and clipped like the rest (clip_gradients then the optimizer, pipeline_flux_lora_1024.rs:691-697).  dev_scale is
 * device memory (eri_adam8_grad_norm_scale_ptr) or NULL for 1. */
int eri_adamw32_step_multi_scaled(const EriAdamW32Tensor *rows, uint32_t n, const EriAdamW32Hyper *hyper, float grad_scale,
                                  const float *dev_scale, void *stream);

/* Exponential moving average of parameters, shadow = decay*shadow + (1-decay)*p in fp32
 * (EMA update, src/trainers/ema_enhanced.rs:79-108), one launch over all rows.
 * `shadow` has the dtype of p. */
typedef struct EriEmaTensor {
    void *shadow;
    const void *p;
    uint64_t numel;
    int32_t dtype_tag;
    int32_t reserved;
} EriEmaTensor;
int eri_ema_update_multi(const EriEmaTensor *rows, uint32_t n, float decay, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* ERI_OPTIM8_H */
