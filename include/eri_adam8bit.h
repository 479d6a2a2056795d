/*
 * eri_adam8bit -- the optimizer objects of EriDiffusion's 8-bit Adam, as a flat C API over
 * eri_optim8.h.  It is the host layer a Rust `impl Adam8bit` (or any other binding) forwards to:
 * it owns the 8-bit states, the step counter and the cached device launch table, and it calls
 * nothing but the functions declared in eri_optim8.h.
 *
 * Two flavours, as in the reference:
 *   EriAdam8bit    step() over a list of parameters that carry their gradients
 *                  (src/trainers/adam8bit_enhanced.rs:160-369)
 *   EriAdam8bitFn  per-tensor update(name, param, grad) keyed by name
 *                  (src/trainers/adam8bit.rs:49-345)
 * Return values follow eri_optim8.h: 0, a positive hipError_t, or a negative EriStatus;
 * eri_last_error() holds the message.  Optimizer-level failures use the reference's wording
 * ("Empty tensor for quantization", "Failed to read optimizer: ...", "Failed to deserialize
 * optimizer: ...", adam8bit_enhanced.rs:46-50,351-357).
 */
#ifndef ERI_ADAM8BIT_H
#define ERI_ADAM8BIT_H

#include "eri_optim8.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---- Parameter: a shared handle to a device tensor and its current gradient ------------------
 * Stands where flame_core::Parameter stands in the reference (tensor(), grad(), apply_update()):
 * the trainer and the optimizer hold the same handle, the optimizer updates the tensor in place.
 * The handle never owns the device memory it points to (crates/core/tests/wrap_external.rs:25-30). */
typedef struct EriParameter EriParameter;
int eri_param_create(void *data, uint64_t numel, int dtype_tag, EriParameter **out);
int eri_param_set_grad(EriParameter *param, const void *grad); /* NULL = no gradient this step; dtype of the parameter */
/* A gradient of another dtype than its parameter: ERI_DTYPE_F32 for a BF16 parameter.  The reference casts
 * every gradient to F32 and never rounds it (adam8bit_enhanced.rs:231-235), so such a gradient enters the
 * step as it is. */
int eri_param_set_grad_typed(EriParameter *param, const void *grad, int grad_dtype_tag);
int eri_param_set_data(EriParameter *param, void *data);       /* Parameter::set_data */
int eri_param_retain(EriParameter *param);                     /* Parameter::clone */
int eri_param_release(EriParameter *param);

/* ---- Adam8bitConfig (adam8bit_enhanced.rs:372-395) ------------------------------------------- */
typedef struct EriAdam8bitConfig {
    double lr;                    /* 1e-3 */
    double beta1, beta2;          /* 0.9, 0.999 */
    double eps;                   /* 1e-8 */
    double weight_decay;          /* 0.01 */
    int32_t amsgrad;              /* false; carried, not used (the reference never reads it) */
    int32_t block_wise;           /* true; the state format here is always block-wise */
    uint64_t percentile_clipping; /* 99; carried, the block-wise format does not clip */
} EriAdam8bitConfig;
void eri_adam8bit_config_default(EriAdam8bitConfig *cfg);

/* ---- Adam8bit: step() over a parameter list --------------------------------------------------- */
typedef struct EriAdam8bit EriAdam8bit;
typedef struct EriEmaModel EriEmaModel; /* declared in full further down */
/* Adam8bit::new(params, config) :161.  `stream` (NULL = default) is used by every later call. */
int eri_adam8bit_new(EriParameter *const *params, uint32_t n, const EriAdam8bitConfig *cfg, void *stream,
                     EriAdam8bit **out);
int eri_adam8bit_destroy(EriAdam8bit *opt);
/* step() :202-291.  Parameters without a gradient are skipped ("Warning: No gradient for
 * param_N" on stderr, :237-240); `skipped`, if not NULL, receives how many. */
int eri_adam8bit_step(EriAdam8bit *opt, uint32_t *skipped);
int eri_adam8bit_zero_grad(EriAdam8bit *opt);                               /* :294 */
double eri_adam8bit_current_lr(const EriAdam8bit *opt);                     /* :302 */
int eri_adam8bit_set_learning_rate(EriAdam8bit *opt, double lr);            /* :307 */
uint64_t eri_adam8bit_quantized_memory_usage(const EriAdam8bit *opt);       /* :312 */
uint64_t eri_adam8bit_get_step(const EriAdam8bit *opt);
/* Extras the trainers apply around the step, folded into it here:
 * a global clip factor (pipeline_flux_lora_sequential.rs:1198-1213) and a per-parameter gradient
 * multiplier (:759-766).  1.0 switches either off. */
int eri_adam8bit_set_grad_scale(EriAdam8bit *opt, float scale);
int eri_adam8bit_set_param_grad_scale(EriAdam8bit *opt, uint32_t index, float scale);
/* ERI_ADAM8_FLAG_* for the steps to come (the whole set, not a bit at a time).  A new optimizer starts with
 * ERI_ADAM8_FLAG_EXACT_PARAM: BF16 parameters come out bit for bit as the reference's chain of rounded fp32
 * operations gives them (F32 parameters and the 8-bit states always do), as the functional flavour's updates
 * always do.  0 selects the faster arithmetic, within one BF16 unit in the last place of those bits per step
 * (0.6-0.9 % faster on a twelve-billion-parameter set). */
int eri_adam8bit_set_flags(EriAdam8bit *opt, uint32_t flags);
/* ERI_ADAM8_MODE_ERI (default: the reference's update) or ERI_ADAM8_MODE_BNB for later steps. */
int eri_adam8bit_set_mode(EriAdam8bit *opt, int mode);
/* EMA inside the step.  With a model attached, every eri_adam8bit_step also performs that model's
 * update(params) (ema_enhanced.rs:79-104: step += 1, shadow = d*shadow + (1-d)*param with d = current_decay(),
 * a name seen for the first time gets a copy of its parameter) over all n parameters of the optimizer, names[i]
 * being the model's name for parameter i -- so the trainer's separate ema.update() call and its sweep go
 * away.  For parameters that take the 8-bit step the shadow is updated by that same launch
 * (ERI_ADAM8_FLAG_EMA); parameters without a gradient, or with fp32 moments, get the plain sweep.  The model is
 * not owned and must outlive the optimizer or be detached (ema = NULL); both must use the same stream. */
int eri_adam8bit_attach_ema(EriAdam8bit *opt, EriEmaModel *ema, const char *const *names, uint32_t n);
/* States that do not exist yet (they are created at the first step that meets their parameter) come out of
 * `lane` of a memory pool (eri_hip_pool_create, include/eri_optim8.h) instead of allocations of their own:
 * a lane 32 GiB or more away from the parameters' makes every later step 10-17 % faster on tables that do not
 * span that much by themselves.  The pool is not owned and must outlive the optimizer (a state that is replaced
 * or destroyed gives its piece back with eri_hip_pool_release, so loading a checkpoint into an optimizer that
 * has stepped does not grow the lane beyond two sets of states); NULL goes back to separate allocations.  No
 * counterpart in the reference, whose states are host vectors. */
int eri_adam8bit_set_state_pool(EriAdam8bit *opt, EriHipPool *pool, uint32_t lane);
/* min_8bit_size (pipeline_flux_lora_1024.rs:451, the policy of the library the state format comes from):
 * from the next step on, a parameter with fewer than `numel` elements that has no 8-bit state yet keeps
 * fp32 moments instead and takes the same update, adam8bit_enhanced.rs:252-275, without the quantiser --
 * one extra launch of the 32-bit step (eri_adamw32_step_multi) over all such parameters, with the
 * bias-corrected step size as its learning rate.  0 (the default) keeps every parameter in the 8-bit
 * format.  Such parameters need gradients of their own dtype and mode ERI (a step in another mode is refused
 * before anything runs).  The loss scale, the per-parameter multipliers and the clip factor reach them as they
 * reach the 8-bit parameters, and the global norm behind the clip factor covers the gradients of both kinds
 * (the trainer that sets min_8bit_size clips every trainable gradient, pipeline_flux_lora_1024.rs:691-697).
 * save_state / load_state carry the fp32 moments as `optimizer.param_N.m32` / `.v32`. */
int eri_adam8bit_set_min_8bit_size(EriAdam8bit *opt, uint64_t numel);
/* Device pointers of one parameter's fp32 moments (NULL if it has none). */
int eri_adam8bit_state32_ptrs(const EriAdam8bit *opt, uint32_t index, float **m, float **v);
/* Global-norm clipping inside step(): max_norm > 0 makes every step first reduce the gradients' global
 * L2 norm on the device (eri_adam8_grad_norm) and apply max_norm / (norm + denom_eps) when the norm is
 * above max_norm -- the trainers' clip_gradients (pipeline_flux_lora_sequential.rs:737,1198-1213)
 * without its per-tensor host reads and gradient rewrites.  max_norm <= 0 switches it off. */
int eri_adam8bit_set_max_grad_norm(EriAdam8bit *opt, float max_norm, float denom_eps);
/* Norm and clip factor of the last step that clipped (waits for the optimizer's stream). */
int eri_adam8bit_last_grad_norm(EriAdam8bit *opt, float *norm, float *scale);
/* NaN / infinite gradient elements seen by the norm pass of the last step that clipped (same wait). */
int eri_adam8bit_last_nonfinite_grads(EriAdam8bit *opt, uint64_t *count);
/* quantization_stats() :318-327: mean over parameters of the mean absolute quantisation error of the
 * first and second moments at the last step.  Tracking costs one extra read pass per step, so it is
 * opt-in: eri_adam8bit_track_quantization_error(opt, 1) before the steps of interest. */
int eri_adam8bit_track_quantization_error(EriAdam8bit *opt, int enabled);
int eri_adam8bit_quantization_stats(EriAdam8bit *opt, float *m_error, float *v_error);
/* save_state / load_state :330-368.  The file is a safetensors container with, per parameter that
 * has state, `optimizer.param_N.m` / `.v` (U8 codes) and `.absmax_m` / `.absmax_v` (F32), and the
 * step counter and learning rate in its metadata. */
int eri_adam8bit_save_state(EriAdam8bit *opt, const char *path);
int eri_adam8bit_load_state(EriAdam8bit *opt, const char *path);
/* Imports a state file written by the reference's own save_state (:330-347): bincode 1.x, default
 * options, of OptimizerState { step: usize, first_moments, second_moments: HashMap<String,
 * QuantizedTensor { quantized_data: Vec<i8>, scale: f32, zero_point: i8, shape: Vec<usize>,
 * quantization_error: f32 }>, learning_rate: f64 } (:30-38,398-404), keys "param_N" (:226).  Each
 * tensor is dequantised as the reference does, (q - zero_point) * scale with non-finite values set
 * to 0 (:117-129), and re-quantised into the blockwise format.  No file of that format ships with
 * the reference, so the layout follows bincode's documented defaults (little-endian, u64 lengths). */
int eri_adam8bit_load_legacy_state(EriAdam8bit *opt, const char *path);
/* Device pointers of one parameter's state (NULL before its first step). */
int eri_adam8bit_state_ptrs(const EriAdam8bit *opt, uint32_t index, uint8_t **m, uint8_t **v, float **absmax_m,
                            float **absmax_v);

/* ---- functional flavour ------------------------------------------------------------------------ */
typedef struct EriAdam8bitFn EriAdam8bitFn;
/* Adam8bit::with_params(lr, beta1, beta2, eps, wd), adam8bit.rs:69-86 */
int eri_adam8bit_fn_with_params(double lr, double beta1, double beta2, double eps, double weight_decay, void *stream,
                                EriAdam8bitFn **out);
int eri_adam8bit_fn_destroy(EriAdam8bitFn *opt);
/* update(name, param, grad) -> new tensor, :101-208.  `param` is left untouched, the new values are
 * written to `out` (numel elements of the same dtype; it may be `param` itself: in-place).  The kernel
 * reads `param` and writes `out`; nothing is copied.  `grad_dtype_tag` is `dtype_tag`, or ERI_DTYPE_F32
 * for BF16 parameters (adam8bit.rs:110 casts the gradient to F32 and does not round it).  Pointers
 * 16-byte aligned.
 * By default every call is one kernel launch and `out` is valid in stream order when the call returns, as
 * the reference's callers may assume (pipeline_sdxl_lora.rs:708-724 reads the new tensor at once). */
int eri_adam8bit_fn_update(EriAdam8bitFn *opt, const char *name, const void *param, const void *grad, uint64_t numel,
                           int dtype_tag, int grad_dtype_tag, void *out);
/* As eri_adam8bit_set_state_pool: states of names not seen yet come out of `lane` of the pool. */
int eri_adam8bit_fn_set_state_pool(EriAdam8bitFn *opt, EriHipPool *pool, uint32_t lane);
/* Batching: with it enabled, update() only queues its row, and ONE launch over all queued rows runs at the
 * next eri_adam8bit_fn_step (which every trainer calls right after its loop of updates:
 * pipeline_flux_lora_sequential.rs:749-794), eri_adam8bit_fn_flush, set_lr, state read or destroy.  Until
 * then `out` is not written and `param` / `grad` must stay alive and unchanged -- a caller that reads the
 * returned tensor, or frees the gradient, before step() must not enable it.  A second update of the same
 * name flushes the first.  The launch tables of the last two distinct sets of rows are kept between flushes:
 * update() returns a new tensor per call (adam8bit.rs:205-207), so a trainer's rows alternate between two
 * sets of addresses, and from the third flush on nothing is uploaded; the same tensors at addresses not seen
 * in the last two flushes cost one small upload.  The hundreds of launches of a LoRA step become one. */
int eri_adam8bit_fn_set_batching(EriAdam8bitFn *opt, int enabled);
int eri_adam8bit_fn_flush(EriAdam8bitFn *opt);
/* How many launches over queued rows have run, and how many of them had to build or re-upload a launch table
 * first (the others found their rows in one of the two tables kept).  Either pointer may be NULL. */
int eri_adam8bit_fn_table_stats(const EriAdam8bitFn *opt, uint64_t *flushes, uint64_t *uploads);
/* n updates in one call and one launch, whatever the batching setting: update(names[i], params[i], grads[i])
 * -> outs[i] for every i (update_params_8bit, adam8bit.rs:333-345, without its loop of launches).
 * grad_dtype_tags may be NULL (every gradient has the dtype of its parameter).  Rows queued earlier run
 * first.  Every row is validated, and the states of names not seen before are created, before anything of
 * the call is launched: if a row is refused or a state cannot be allocated, nothing of the call runs and no
 * state of the call stays behind.  A name that repeats within the call splits it there: the rows up to the
 * repetition are one launch, the rest the next (two updates of one tensor are two steps of its state). */
int eri_adam8bit_fn_update_many(EriAdam8bitFn *opt, const char *const *names, const void *const *params,
                                const void *const *grads, const uint64_t *numels, const int32_t *dtype_tags,
                                const int32_t *grad_dtype_tags, void *const *outs, uint32_t n);
int eri_adam8bit_fn_step(EriAdam8bitFn *opt);                   /* :89-92: runs what is queued, bumps the counter */
int eri_adam8bit_fn_set_lr(EriAdam8bitFn *opt, float lr);       /* :95-98 */
uint64_t eri_adam8bit_fn_get_step(const EriAdam8bitFn *opt);    /* :311-313 */
/* memory_stats() :253-266: number of named states and their bytes */
int eri_adam8bit_fn_memory_stats(const EriAdam8bitFn *opt, uint64_t *num_params, uint64_t *bytes);
/* get_state_as_tensors / load_state_from_tensors :296-329, one name at a time: fp32 moments.
 * `numel` of an unknown name reads 0.  m_out / v_out and m / v are DEVICE buffers of numel floats (the
 * reference hands out and takes device tensors): the conversion runs on the optimizer's stream, and the
 * buffers are valid in stream order; ordinary host memory is refused (ERI_ERR_ARG). */
int eri_adam8bit_fn_state_numel(const EriAdam8bitFn *opt, const char *name, uint64_t *numel);
int eri_adam8bit_fn_get_state_fp32(EriAdam8bitFn *opt, const char *name, float *m_out, float *v_out);
int eri_adam8bit_fn_load_state_fp32(EriAdam8bitFn *opt, const char *name, const float *m, const float *v,
                                    uint64_t numel);

/* ---- small host-side helpers that live beside the optimizers in the reference -------------------- */

/* analyze_optimizer_memory(num_params, precision), adam8bit_enhanced.rs:406-431: the reference's coarse
 * accounting (fp32 parameters; states of 8, 4, 2 or 1 bytes per parameter for "fp32", "fp16", "8bit",
 * "4bit"; anything else counts as fp32 with the description "Unknown precision").
 * memory_reduction_percent is against fp32 states and is absent (has_reduction = 0) for "fp32". */
typedef struct EriOptimizerMemoryReport {
    uint64_t num_params;
    double param_memory_gb, state_memory_gb, total_memory_gb;
    double memory_reduction_percent;
    int32_t has_reduction;
    char description[44];
} EriOptimizerMemoryReport;
int eri_analyze_optimizer_memory(uint64_t num_params, const char *precision, EriOptimizerMemoryReport *out);

/* ---- EMAModel (src/trainers/ema_enhanced.rs:12-204): shadow copies of named parameters ----------------
 * The shadows live in device memory owned by the object; update() is one eri_ema_update_multi launch
 * over every parameter already known, plus a device copy for names seen for the first time (:100-103).
 * eri_ema_new: decay outside (0, 1] is refused with "EMA decay must be in (0, 1], got ..." (:36-41);
 * the reference's defaults are use_bias_correction = 1, power = 1 (:48-50; with_config :55-64). */
int eri_ema_new(float decay, int use_bias_correction, float power, void *stream, EriEmaModel **out);
int eri_ema_destroy(EriEmaModel *ema);
/* init_from_params :67-76: every shadow becomes a copy of its parameter. */
int eri_ema_init_from_params(EriEmaModel *ema, const char *const *names, EriParameter *const *params, uint32_t n);
/* update :79-104: step += 1, then shadow = d*shadow + (1-d)*param with d = current_decay(). */
int eri_ema_update(EriEmaModel *ema, const char *const *names, EriParameter *const *params, uint32_t n);
/* copy_to :130-142: parameter memory <- shadow; an unknown name answers
 * "No EMA weights found for parameter: ..." and nothing is copied. */
int eri_ema_copy_to(EriEmaModel *ema, const char *const *names, EriParameter *const *params, uint32_t n);
uint64_t eri_ema_step(const EriEmaModel *ema);             /* :175 */
int eri_ema_set_step(EriEmaModel *ema, uint64_t step);     /* :180 */
float eri_ema_current_decay(const EriEmaModel *ema);       /* :185 */
uint32_t eri_ema_num_shadows(const EriEmaModel *ema);
/* shadow_params() :170, one name at a time: device pointer, element count and dtype of a shadow. */
int eri_ema_shadow(const EriEmaModel *ema, const char *name, void **data, uint64_t *numel, int *dtype_tag);

/* EMA decay helpers, src/trainers/ema_enhanced.rs:268-279 and compute_effective_decay :106-127
 * (power schedule over the first 1000 steps, optional bias correction below step 1000).  The value
 * they give is what a trainer passes to eri_ema_update_multi. */
float eri_ema_decay_from_half_life(uint64_t half_life_steps);
float eri_ema_decay_from_window(uint64_t window_size);
float eri_ema_effective_decay(float decay, uint64_t step, float power, int use_bias_correction);

#ifdef __cplusplus
}
#endif
#endif /* ERI_ADAM8BIT_H */
