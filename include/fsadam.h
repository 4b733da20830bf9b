/*
 * fsadam -- C ABI of the MI355X (gfx950) fused multi-tensor Adam step.
 *
 * This header is the drop-in boundary for the one native entry point of fairscale,
 *     fairscale.fused_adam_cuda.adam(chunk_size, noop_flag, tensor_lists, lr, beta1, beta2, eps,
 *                                    grad_scale, optim_scale, found_inf, step, mode,
 *                                    bias_correction, decay)
 * (pybind definition: fairscale/clib/fused_adam_cuda/fused_adam_cuda.cpp:4-8, call site:
 * fairscale/optim/adam.py:261-276).  Everything is plain pointers, sizes and C scalars: no torch,
 * no C++ types, no exceptions cross it.  All device pointers are borrowed and updated in place;
 * all work is enqueued on the caller's hipStream_t and nothing here synchronises the host with it.
 *
 * Return convention: 0 on success, a negative FSADAM_E* code on failure; the message for the last
 * failure on the calling thread is available from fsadam_last_error().
 */
#ifndef FSADAM_H_
#define FSADAM_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FSADAM_ABI_VERSION 4

/* Precision modes = the four dtype combinations the reference dispatches on
 * (fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:172-256; Python enum
 * fairscale/optim/adam.py:19-23).                         p      g      m,v    p_copy            */
#define FSADAM_FULL_PRECISION 0                         /* f32    f32    f32    -                 */
#define FSADAM_MIXED_PRECISION 1                        /* f32    f16    f32    f16 (written)     */
#define FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION 2       /* f16    f16    f32    -                 */
#define FSADAM_PURE_FP16 3                              /* f16    f16    f16    -   (state*scale) */
/* Not a combination the reference dispatches on: the fp32 step of an FSDP shard with the fp16 copy of
 * the parameters written in the same pass -- what FullyShardedDataParallel._cast_fp32_param_shards_to_fp16
 * (fairscale/nn/data_parallel/fully_sharded_data_parallel.py:2253-2267) recomputes before the next
 * forward: p_copy = half(p), one rounding of the stored fp32 value (kernel.cu:114,129).              */
#define FSADAM_FULL_PRECISION_FP16_COPY 4               /* f32    f32    f32    f16 (written)     */

/* eps placement (adamMode_t, fused_adam_cuda_kernel.cu:16-19) */
#define FSADAM_EPS_INSIDE_SQRT 0
#define FSADAM_EPS_OUTSIDE_SQRT 1

#define FSADAM_OK 0
#define FSADAM_EINVAL (-1)   /* bad argument (NULL pointer, unknown mode, negative size ...)         */
#define FSADAM_EHIP (-2)     /* a HIP runtime call or the kernel launch failed                      */
#define FSADAM_ENOMEM (-3)   /* host or device allocation of the tensor table failed                */
#define FSADAM_ENODEVICE (-4) /* no usable gfx950 device                                            */

/* One row of the tensor list: replaces column t of the reference's tensor_lists[d][t]
 * (TensorListMetadata, fairscale/clib/fused_adam_cuda/multi_tensor_apply.cuh:18-25).  numel is
 * 64-bit (the reference truncates to int, multi_tensor_apply.cuh:21,80).  Every pointer must address
 * numel contiguous elements of the dtype the mode implies.  p_copy is used only by the two modes that
 * write an fp16 copy (MIXED_PRECISION, FULL_PRECISION_FP16_COPY). */
typedef struct FsAdamTensor {
    void* p;        /* parameters (fp32 master copy in MIXED)                       */
    void* m;        /* exp_avg                                                      */
    void* v;        /* exp_avg_sq                                                   */
    const void* g;  /* gradients                                                    */
    void* p_copy;   /* copy-out modes: fp16 parameters to overwrite; else ignored    */
    int64_t numel;
} FsAdamTensor;

typedef struct FsAdamPlan FsAdamPlan; /* opaque: a device-resident tensor table + launch geometry */

/* What a plan looks like after fsadam_plan_set_tensors (host-side bookkeeping, for tests/benches). */
typedef struct FsAdamPlanInfo {
    int32_t mode;
    int32_t device;
    int64_t n_tensors;
    int64_t total_elems;
    int64_t tile_elems;        /* elements one workgroup handles                                        */
    int64_t large_chunk_elems; /* elements per shared descriptor of a large tensor                      */
    int64_t n_descriptors;     /* 64-byte rows of the device table                                      */
    int64_t n_vector_tensors;  /* tensors whose every stream is aligned to its 64/128-bit vector         */
    int64_t n_scalar_tensors;  /* tensors with a stream that is only element-aligned                    */
    int64_t n_launches;        /* kernel launches per step: 0 or 1                                      */
    int64_t grid;              /* workgroups per step, all launches                                     */
    int64_t block;             /* threads per workgroup                                                 */
    int64_t lds_throttle;      /* bytes of LDS ballast per workgroup                                    */
    int64_t uploads;           /* how many times the table has been (re)sent to the device              */
    int64_t n_runs;            /* rows the layout works on: non-empty tensors after merging (option merge_runs) */
} FsAdamPlanInfo;

/* How fsadam_plan_set_tensors would cut a tensor list into descriptors (see fsadam_layout). */
typedef struct FsAdamLayout {
    int64_t tile_elems;
    int64_t large_chunk_elems;
    int64_t n_large_tensors;     /* numel >= 131072: descriptors shared by large_chunk_elems/tile_elems tiles */
    int64_t n_small_tensors;     /* under mid_chunk_elems: one descriptor per tile                            */
    int64_t n_empty_tensors;     /* numel == 0: skipped                                                       */
    int64_t n_large_descriptors;
    int64_t n_small_descriptors;
    int64_t grid_large;          /* workgroups of the large tensors (some past a tensor's end: they exit)       */
    int64_t grid_small;          /* workgroups with a descriptor of their own                                  */
    int64_t mid_chunk_elems;     /* elements per shared descriptor of a middle-sized tensor; 0: no such class   */
    int64_t n_mid_tensors;       /* mid_chunk_elems <= numel < 131072                                          */
    int64_t n_mid_descriptors;
    int64_t grid_mid;            /* workgroups of the middle-sized tensors                                     */
    int64_t n_runs;              /* non-empty tensors after merging; the three n_*_tensors above count these    */
} FsAdamLayout;

/* ---- library ---- */

/* FSADAM_ABI_VERSION the library was built with. */
int fsadam_version(void);

/* Message of the last failure on this thread ("" if none).  Never NULL; valid until the next call. */
const char* fsadam_last_error(void);

/* Host-only.  The step size exactly as the reference's dispatcher rounds it
 * (fused_adam_cuda_kernel.cu:153-162): bias corrections through double pow then narrowed to float,
 * lr*sqrtf(bc2)/bc1 in float; lr when bias_correction != 1. */
float fsadam_step_size(float lr, float beta1, float beta2, int step, int bias_correction);

/* Tuning knobs, by name; returns FSADAM_EINVAL for an unknown name or a value out of range.
 *   "lds_throttle"  bytes of untouched LDS given to every workgroup, which caps how many workgroups
 *                   share a compute unit (LDS is handed out in granules of 1280 bytes, 128 per compute unit:
 *                   B bytes allow floor(128 / ceil(B / 1280)) workgroups); 0 = no cap, -1 (default) = chosen
 *                   by precision mode and list size (11-15 KiB: 10 waves per compute unit in the 28-byte
 *                   modes, 12 in the others, one step more for small lists)
 *   "merge_runs"    1 (default): consecutive rows of a list that continue each other in every stream (p, m, v, g and
 *                   the fp16 copy each start where the row before ended: parameters that are back-to-back views of
 *                   one buffer, with gradients and state laid out alike) are laid out as ONE tensor, so that a
 *                   list of views into flat buffers costs what the flat buffers cost; 0: every row on its own
 *   "align_heads"   1 (default): a tensor of 8192 elements or more whose streams start off a 128-byte line (a view
 *                   into a flat buffer) gives its first elements, at most 511, to a short descriptor of their own, so
 *                   that every tile behind them starts on line boundaries (see fsadam_head_elems); 0: tiles start
 *                   at element 0 wherever that is (lists of packed views measured 20 % slower)
 *   "mid_tiles"     tiles that share one descriptor of a middle-sized tensor (one of at least mid_tiles tiles and
 *                   under 131072 elements): 0 (every such tile has its own descriptor) or a power of two up to 64
 *                   (default 16).  Shared descriptors make the table of a many-tensor list 10x shorter, which is
 *                   what is sent again when a pointer of the list moves
 *   "upload_stream" (tables of more than 48 rows; a shorter one travels in the arguments of one small launch on the
 *                   caller's stream)  1 (default): a new descriptor table is copied to the device on a stream the library owns,
 *                   and the caller's stream waits for that copy's event, so the copy overlaps the step still
 *                   running on the caller's stream; 0: the copy is enqueued on the caller's stream
 *   "grad_items"    gradient pass: 16-byte vectors per lane, 2, 4 or 8; 0 = 8 for a read-only pass,
 *                   4 for one that writes the gradients back (default 0)
 *   "grad_lds_throttle"  gradient pass: LDS ballast per workgroup in bytes; -1 = 14080 / 12800 likewise
 *   "grad_waves"    gradient pass: tiles (one wave each) per workgroup, 1, 4 or 16; the workgroup writes one
 *                   partial result.  0 = 1 for either kind of pass (default 0)
 * A workgroup of the step is one wave64 handling one vector per lane and stream, tiles are taken in dispatch order
 * and full tiles of streams that are only element-aligned use the same vector instructions: the alternatives
 * (128/256 threads, two vectors per lane, an XCD-aware tile order, element-wise tiles, smaller shared chunks)
 * were measured no faster or slower and are not offered.
 * Affects plans whose tensors are set after the call. */
int fsadam_set_option(const char* name, int64_t value);
int fsadam_get_option(const char* name, int64_t* value);

/* ---- the step: replaces fairscale.fused_adam_cuda.adam (fused_adam_cuda.cpp:4-8 /
 * fused_adam_cuda(), fused_adam_cuda_kernel.cu:137-265 / multi_tensor_apply<depth>(),
 * multi_tensor_apply.cuh:40-130).
 *
 * tensors/n_tensors : host array, one row per tensor of the list (n_tensors >= 1; rows with numel 0
 *                     are skipped).  The reference's chunk_size and noop_flag arguments have no
 *                     counterpart: chunking is internal and the reference never reads noop_flag
 *                     (fused_adam_cuda_kernel.cu:26).
 * scalars           : C floats, i.e. already narrowed the way pybind narrows Python floats.
 * found_inf_dev     : device float[1]; set to 1.0f (never cleared) when a stored fp16 m or v is
 *                     non-finite.  Only PURE_FP16 can set it (fused_adam_cuda_kernel.cu:103-105);
 *                     may be NULL in the other modes.
 * hip_stream        : hipStream_t to enqueue on (NULL = the default stream).
 *
 * The device-side tensor table is cached inside the library, keyed on the contents of `tensors`;
 * an unchanged list costs no upload.
 *
 * Not recordable into a HIP graph: the step size depends on `step` and travels by value, so a replay
 * would repeat the recorded step's bias correction.  A call on a stream that is being captured
 * returns FSADAM_EINVAL and enqueues nothing (the same holds for the plan calls and the gradient pass). */
int fsadam_step(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, float lr, float beta1,
                float beta2, float eps, float grad_scale, float optim_scale, float decay, int step,
                int eps_mode, int bias_correction, float* found_inf_dev, void* hip_stream);

/* ---- explicit plans: same step, table lifetime owned by the caller (what the Python optimizer
 * uses so that an OSS/FSDP shard's table is built once and re-sent only when a pointer moves).
 * A plan belongs to the device that was current at its first fsadam_plan_set_tensors and must not
 * be used by two threads at once.  fsadam_plan_set_tensors may be called while earlier steps of the
 * plan are still running: tables rotate through a ring of three, and the call only waits for the
 * step that last used the slot it is about to overwrite. */
int fsadam_plan_create(int precision_mode, FsAdamPlan** out);
int fsadam_plan_set_tensors(FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n_tensors, void* hip_stream);
int fsadam_plan_step(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, float grad_scale,
                     float optim_scale, float decay, int step, int eps_mode, int bias_correction,
                     float* found_inf_dev, void* hip_stream);
int fsadam_plan_info(const FsAdamPlan* plan, FsAdamPlanInfo* out);
/* on = 0 (default): an event is recorded behind every step of the plan; it is what the library waits for before it
 * overwrites a table a step may still read, and what orders a call on another stream behind the one before.
 * on = 1: the event is only recorded when one of those needs it, which makes a step 3 us shorter, but touches the
 * stream after the call that used it has returned: every stream passed to this plan must then stay alive until
 * fsadam_plan_destroy.  (The Python binding switches it on for its plans: torch's streams live as long as the
 * process.  fsadam_step and fsadam_grad_pass always record.) */
int fsadam_plan_lazy_events(FsAdamPlan* plan, int on);
int fsadam_plan_destroy(FsAdamPlan* plan);

/* Sets m and v of every tensor in the plan's current table to zero, in one launch over the step's own layout: what
 * follows an overflow of the fp16 state, where fairscale/optim/adam.py:285-288 re-allocates exp_avg / exp_avg_sq of
 * every parameter (a foreach over the 582 state tensors of a Llama-7B list takes 70 ms, this launch 5).  The
 * parameters and gradients are not touched.  Enqueued on hip_stream like a step; not recordable into a graph. */
int fsadam_plan_zero_state(FsAdamPlan* plan, void* hip_stream);

/* As fsadam_plan_step, with the gradient scale read by the kernel from device memory (one float that must be
 * valid when the kernel runs; nothing is synchronised on the host).  For callers that compute the scale
 * on the device: a clip factor max(1, norm / max_norm) from fsadam_grad_pass's sum of squares, or a loss
 * scale kept in a device tensor.  The result has the bits fsadam_plan_step gives for a host float of
 * the same value.  No counterpart in the reference, whose grad_scale is a host float
 * (fused_adam_cuda.cpp:4, fused_adam_cuda_kernel.cu:143). */
int fsadam_plan_step_dev_scale(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, const float* grad_scale_dev,
                               float optim_scale, float decay, int step, int eps_mode, int bias_correction,
                               float* found_inf_dev, void* hip_stream);

/* Host-only planning (no device needed): how the list would be laid out under the current options.
 * tensor_class[n_tensors] (may be NULL): 0 empty, 1 small, 2 large, 3 middle-sized.  vector_ok[n_tensors] (may be
 * NULL): 1 = every stream aligned to its 64/128-bit vector.  With option merge_runs a tensor is laid out with
 * the run of consecutive tensors it belongs to: class, alignment and head are the run's. */
int fsadam_layout(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, FsAdamLayout* out,
                  uint8_t* tensor_class, uint8_t* vector_ok);

/* Host-only: how many leading elements of this tensor the layout gives to a short descriptor of their own so
 * that the tiles behind them start where the streams meet 128-byte lines (and 1 KiB boundaries where they
 * can): 0 for tensors under 8192 elements, for streams that are aligned already, when no count improves the
 * alignment, and with option "align_heads" = 0; at most 511 otherwise.  The head's descriptors are counted
 * among the small ones of fsadam_layout, and the tensor's class and vector_ok refer to what follows the head.
 * The values a step writes do not depend on it.  No counterpart in the reference, whose chunks always start
 * at element 0 (multi_tensor_apply.cuh:74-86). */
int fsadam_head_elems(const FsAdamTensor* tensor, int precision_mode, int64_t* head);

/* ---- gradient pass: what runs on the gradients BEFORE the step, in one read.
 * Replaces, for one rank's gradients on one device:
 *   torch._amp_foreach_non_finite_check_and_unscale_(grads, found_inf, inv_scale)
 *       as called by fairscale/optim/grad_scaler.py:211-215 (and by torch's GradScaler, which
 *       fairscale.optim.GradScaler subclasses, grad_scaler.py:60-68), and
 *   calc_grad_norm(parameters, p) for p = 2 and p = inf, fairscale/internal/params.py:59-76, the
 *       local norm behind OSS.clip_grad_norm (fairscale/optim/oss.py:244-302) and
 *       FullyShardedDataParallel.clip_grad_norm_ (fully_sharded_data_parallel.py:621-687).
 * inv_scale_dev, when not NULL, is a device float[1] that is read instead of the host value inv_scale
 * (a loss scaler keeps its scale on the device; no host round trip).
 * Per element: found_inf is raised when the incoming g is +-inf/NaN; r = (inv_scale == 1) ? g :
 * dtype(float(g) * inv_scale) is what unscaling stores; sum_squares and abs_max are taken of float(r).
 * write_back != 0 stores r over g (the reference behaviour); write_back == 0 leaves the gradients
 * untouched, for callers that fold the scale into fsadam_step's grad_scale instead.
 * Outputs (device pointers, each may be NULL): found_inf_dev float[1], only ever set to 1.0f;
 * sum_squares_dev double[1] and abs_max_dev float[1], overwritten.  The reductions run in a fixed
 * order: the same inputs give the same bits.  NaN gradients make both norms NaN, as in torch. */
typedef struct FsGradTensor {
    void* g;
    int64_t numel;
} FsGradTensor;

#define FSADAM_GRAD_F32 0
#define FSADAM_GRAD_F16 1

int fsadam_grad_pass(const FsGradTensor* grads, int64_t n_tensors, int grad_dtype, float inv_scale, const float* inv_scale_dev,
                     int write_back, float* found_inf_dev, double* sum_squares_dev, float* abs_max_dev, void* hip_stream);

/* fsadam_grad_pass for callers that cannot allocate device memory: code that runs between the begin and end of
 * a HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference
 * (its gradient passes are torch operators, which allocate their outputs).  Same arguments, same results:
 * what is stored, the flag and the maximum have the bits fsadam_grad_pass gives; the sum of squares agrees
 * within 1e-6 relative (16 tiles share one partial here, each tile has its own there, so the additions group
 * differently).  The call makes no hipMalloc / hipFree / hipHostMalloc, creates no stream or event and copies
 * nothing with the copy engines: the descriptor table travels in kernel arguments (one small launch per 48
 * rows) and lives, with the partial results, in an array that is part of the library's code object,
 * FSADAM_NOALLOC_MAX_DESCRIPTORS * 64 + (FSADAM_NOALLOC_MAX_WORKGROUPS + 521) * 16 bytes (1.26 MiB) per GPU,
 * held until the process ends.  A list that needs more descriptors or workgroups than that is refused with
 * FSADAM_EINVAL (a workgroup covers 65536 fp16 / 32768 fp32 elements when the pass only reads, half as many
 * when it writes back: at least 1.07e9 elements in every case; a tensor of 131072 elements or more takes one
 * descriptor per 2^16..2^24 elements, smaller ones up to 16, plus one for a misaligned start).  Tuning options
 * are not consulted.  All calls on one GPU share that GPU's array: calls whose kernels may overlap (different
 * streams without an order between them, a replaying graph beside an eager call) race; calls on one stream are ordered
 * by it.  The race is not prevented but it is noticed: the first kernel of a call takes possession of the array and the
 * last gives it back, and a call that did not own the array from its beginning to its end reports NaN in all three
 * outputs (a flag that is not zero reads as an overflow, so the step is skipped) instead of numbers that may be wrong;
 * the gradients of a pass that writes back are then undefined.  Lists that overlap in time must be such that either
 * call's kernels may read the other's descriptors; the stream must belong to the current device.  The call may
 * be recorded into a HIP graph (its scalars do not depend on a step count); make the first call on a device outside
 * any capture, since that call looks up the array's address. */
#define FSADAM_NOALLOC_MAX_DESCRIPTORS 4096
#define FSADAM_NOALLOC_MAX_WORKGROUPS 65536
int fsadam_grad_pass_noalloc(const FsGradTensor* grads, int64_t n_tensors, int grad_dtype, float inv_scale, const float* inv_scale_dev,
                             int write_back, float* found_inf_dev, double* sum_squares_dev, float* abs_max_dev, void* hip_stream);

/* Drops the tables cached by fsadam_step and fsadam_grad_pass (synchronises the devices that own them). */
int fsadam_clear_cache(void);

#ifdef __cplusplus
}
#endif
#endif /* FSADAM_H_ */
