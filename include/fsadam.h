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

#define FSADAM_ABI_VERSION 1

/* Precision modes = the four dtype combinations the reference dispatches on
 * (fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:172-256; Python enum
 * fairscale/optim/adam.py:19-23).                         p      g      m,v    p_copy            */
#define FSADAM_FULL_PRECISION 0                         /* f32    f32    f32    -                 */
#define FSADAM_MIXED_PRECISION 1                        /* f32    f16    f32    f16 (written)     */
#define FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION 2       /* f16    f16    f32    -                 */
#define FSADAM_PURE_FP16 3                              /* f16    f16    f16    -   (state*scale) */

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
 * numel contiguous elements of the dtype the mode implies.  p_copy is read only in MIXED mode. */
typedef struct FsAdamTensor {
    void* p;        /* parameters (fp32 master copy in MIXED)                       */
    void* m;        /* exp_avg                                                      */
    void* v;        /* exp_avg_sq                                                   */
    const void* g;  /* gradients                                                    */
    void* p_copy;   /* MIXED: fp16 parameters to overwrite; otherwise ignored/NULL  */
    int64_t numel;
} FsAdamTensor;

typedef struct FsAdamPlan FsAdamPlan; /* opaque: a device-resident tensor table + launch geometry */

/* What a plan looks like after fsadam_plan_set_tensors (host-side bookkeeping, for tests/benches). */
typedef struct FsAdamPlanInfo {
    int32_t mode;
    int32_t device;
    int64_t n_tensors;
    int64_t total_elems;
    int64_t total_chunks;     /* work items of chunk_elems elements (last one of a tensor may be short) */
    int64_t chunk_elems;
    int64_t n_vector_tensors; /* tensors whose every stream is 16-byte aligned: 128-bit path          */
    int64_t n_scalar_tensors; /* tensors taking the element-wise path because of a misaligned stream  */
    int64_t n_launches;       /* kernel launches one step needs (1 unless n_tensors > table window)   */
    int64_t grid;             /* workgroups of the first launch                                       */
    int64_t block;            /* threads per workgroup                                                */
    int64_t uploads;          /* how many times the table has been (re)sent to the device             */
} FsAdamPlanInfo;

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
 *   "chunk_elems"   elements per work item (multiple of 2048, default 16384)
 *   "wg_per_cu"     resident workgroups requested per compute unit (default 8)
 *   "nontemporal"   0/1: non-temporal hint on streaming loads and stores (default 1)
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
 * an unchanged list costs no upload. */
int fsadam_step(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, float lr, float beta1,
                float beta2, float eps, float grad_scale, float optim_scale, float decay, int step,
                int eps_mode, int bias_correction, float* found_inf_dev, void* hip_stream);

/* ---- explicit plans: same step, table lifetime owned by the caller (what the Python optimizer
 * uses so that an OSS/FSDP shard's table is built once and re-sent only when a pointer moves). */
int fsadam_plan_create(int precision_mode, FsAdamPlan** out);
int fsadam_plan_set_tensors(FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n_tensors, void* hip_stream);
int fsadam_plan_step(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, float grad_scale,
                     float optim_scale, float decay, int step, int eps_mode, int bias_correction,
                     float* found_inf_dev, void* hip_stream);
int fsadam_plan_info(const FsAdamPlan* plan, FsAdamPlanInfo* out);
int fsadam_plan_destroy(FsAdamPlan* plan);

/* Host-only planning (no device needed): fills chunk_prefix[n_tensors+1] (exclusive prefix sum of
 * per-tensor chunk counts) and vector_ok[n_tensors] (1 = every stream 16-byte aligned) the way
 * fsadam_plan_set_tensors lays the table out for `chunk_elems`. */
int fsadam_layout(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, int64_t chunk_elems,
                  uint64_t* chunk_prefix, uint8_t* vector_ok);

/* Drops the tables cached by fsadam_step (synchronises the devices that own them). */
int fsadam_clear_cache(void);

/* ---- measurement aid: a plain 128-bit copy kernel of known traffic (nbytes read + nbytes
 * written), used to calibrate the profiler's FETCH_SIZE / WRITE_SIZE counters and as the
 * achievable-bandwidth yardstick next to the Adam kernels.  nbytes must be a multiple of 16 and
 * both pointers 16-byte aligned. */
int fsadam_calib_copy(void* dst, const void* src, int64_t nbytes, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* FSADAM_H_ */
