// Fused multi-tensor Adam step for MI355X (gfx950): kernels + C ABI (include/fsadam.h).
//
// Takes the place of fairscale's one native module:
//   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu   (update equations :94-130, step size :153-162,
//                                                                dtype dispatch :172-256)
//   fairscale/clib/fused_adam_cuda/multi_tensor_apply.cuh      (tensor-list launcher :40-130)
//
// Design, in one paragraph.  The path is elementwise and HBM-bound (14-28 bytes per element, a few
// dozen flops), so there is no MFMA here; the job is to keep every HBM channel busy.  The tensor list
// lives in a device-resident table (one 64-byte row per tensor) that is uploaded once and reused
// every step; an exclusive prefix sum of per-tensor chunk counts turns "work item c" into (tensor,
// chunk) by a binary search that every workgroup runs out of LDS, so ONE launch covers any number
// of tensors (the reference needs one launch per 36 tensors / 320 chunks because its table travels
// by value in the kernel arguments).  Workgroups of four wave64s walk the work items grid-stride;
// inside an item every lane moves 128-bit vectors (two per fp32 stream, one per fp16 stream in the
// half-precision modes) with several independent loads in flight before the first use, does the
// update in fp32 registers, and writes p, m, v (and the fp16 copy of p) back with 128-bit stores.
// Tensors with a stream that is not 16-byte aligned, and the ragged last few elements of a tensor,
// go through an element-wise path with the same arithmetic.
//
// Arithmetic is IEEE float32 exactly as written in the reference source: separate multiplies and
// adds (compiled with -ffp-contract=off), correctly rounded division and square root (hipcc's
// default for fp32), round-to-nearest-even conversions to fp16.  Dividing by a power-of-two scale is
// done as a multiplication by its exact reciprocal, which gives the same bits.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "fsadam.h"

namespace {

// --------------------------------------------------------------------------------------------
// shared host/device definitions
// --------------------------------------------------------------------------------------------

constexpr int kBlock = 256;          // 4 wave64 per workgroup
constexpr int kWindow = 8192;        // tensors whose chunk prefix one launch stages in LDS (32 KiB + 4)
constexpr int kChunkQuantum = 2048;  // chunk_elems granularity: keeps chunk bases 16-byte aligned in every dtype

struct alignas(16) TensorRow {  // 64 bytes
    void* p;
    void* m;
    void* v;
    const void* g;
    void* p_copy;
    int64_t numel;
    uint32_t vector_ok;  // every stream 16-byte aligned
    uint32_t pad;
};
static_assert(sizeof(TensorRow) == 64, "table row must stay 64 bytes");

enum : int { kGradScalePow2 = 1, kOptimScalePow2 = 2 };

struct StepScalars {
    float b1, b2, one_minus_b1, one_minus_b2;
    float eps, decay, step_size;
    float grad_scale, inv_grad_scale;
    float optim_scale, inv_optim_scale;
    int eps_mode;  // 0: sqrt(v+eps), 1: sqrt(v)+eps
    int flags;     // kGradScalePow2 | kOptimScalePow2
};

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// Pointers read out of the tensor table would otherwise be generic (flat_* instructions, which also
// tie up the LDS counter); these live in global memory, so say so.
#define FS_GLOBAL __attribute__((address_space(1)))
template <typename T>
using gptr = FS_GLOBAL T*;

template <int MODE>
struct ModeTraits;
template <>
struct ModeTraits<FSADAM_FULL_PRECISION> {
    using P = float; using G = float; using S = float;
    static constexpr bool kCopy = false, kScaled = false;
    static constexpr int kVec = 4;
};
template <>
struct ModeTraits<FSADAM_MIXED_PRECISION> {
    using P = float; using G = _Float16; using S = float;
    static constexpr bool kCopy = true, kScaled = false;
    static constexpr int kVec = 8;
};
template <>
struct ModeTraits<FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION> {
    using P = _Float16; using G = _Float16; using S = float;
    static constexpr bool kCopy = false, kScaled = false;
    static constexpr int kVec = 8;
};
template <>
struct ModeTraits<FSADAM_PURE_FP16> {
    using P = _Float16; using G = _Float16; using S = _Float16;
    static constexpr bool kCopy = false, kScaled = true;
    static constexpr int kVec = 8;
};

// --------------------------------------------------------------------------------------------
// device code
// --------------------------------------------------------------------------------------------

// N consecutive elements of T held as raw 16-byte quads until they are needed.
template <typename T, int N>
struct Packet {
    static constexpr int kQuads = N * (int)sizeof(T) / 16;
    static_assert(kQuads >= 1 && kQuads * 16 == N * (int)sizeof(T), "packet must be whole 16-byte quads");
    f32x4 q[kQuads];
};

template <typename T, int N, bool NT>
__device__ __forceinline__ Packet<T, N> load_packet(gptr<const T> ptr) {
    Packet<T, N> r;
    gptr<const f32x4> src = reinterpret_cast<gptr<const f32x4>>(ptr);
#pragma unroll
    for (int k = 0; k < Packet<T, N>::kQuads; ++k) {
        if (NT)
            r.q[k] = __builtin_nontemporal_load(src + k);
        else
            r.q[k] = src[k];
    }
    return r;
}

template <typename T, int N, bool NT>
__device__ __forceinline__ void store_packet(gptr<T> ptr, const Packet<T, N>& r) {
    gptr<f32x4> dst = reinterpret_cast<gptr<f32x4>>(ptr);
#pragma unroll
    for (int k = 0; k < Packet<T, N>::kQuads; ++k) {
        if (NT)
            __builtin_nontemporal_store(r.q[k], dst + k);
        else
            dst[k] = r.q[k];
    }
}

template <int N>
__device__ __forceinline__ void unpack(const Packet<float, N>& r, float (&out)[N]) {
#pragma unroll
    for (int k = 0; k < N; ++k) out[k] = r.q[k / 4][k % 4];
}
template <int N>
__device__ __forceinline__ void unpack(const Packet<_Float16, N>& r, float (&out)[N]) {
#pragma unroll
    for (int k = 0; k < N / 8; ++k) {
        const f16x8 h = __builtin_bit_cast(f16x8, r.q[k]);
#pragma unroll
        for (int e = 0; e < 8; ++e) out[k * 8 + e] = (float)h[e];  // exact
    }
}
template <int N>
__device__ __forceinline__ void pack(const float (&in)[N], Packet<float, N>& r) {
#pragma unroll
    for (int k = 0; k < N; ++k) r.q[k / 4][k % 4] = in[k];
}
// float -> half, round to nearest even (v_cvt_f16_f32 under the default rounding mode).
// Returns true when a produced half is +-inf or NaN.
template <int N>
__device__ __forceinline__ bool pack(const float (&in)[N], Packet<_Float16, N>& r) {
    bool bad = false;
#pragma unroll
    for (int k = 0; k < N / 8; ++k) {
        f16x8 h;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            h[e] = (_Float16)in[k * 8 + e];
            const uint16_t bits = __builtin_bit_cast(uint16_t, h[e]);
            bad |= ((bits & 0x7c00u) == 0x7c00u);
        }
        r.q[k] = __builtin_bit_cast(f32x4, h);
    }
    return bad;
}

// The update for one element, all in fp32 registers.
//   unscaled state: fused_adam_cuda_kernel.cu:115-130     scaled (fp16) state: :94-114
// out_m/out_v are what gets STORED (already multiplied by optim_scale when kScaled).
template <bool kScaled>
__device__ __forceinline__ void adam_update(const StepScalars& s, float in_p, float in_m, float in_v, float in_g,
                                            float& out_p, float& out_m, float& out_v) {
    const float scaled_grad = (s.flags & kGradScalePow2) ? in_g * s.inv_grad_scale : in_g / s.grad_scale;
    float momentum, velocity;
    if (kScaled) {
        const bool pow2 = (s.flags & kOptimScalePow2) != 0;
        const float m_un = pow2 ? in_m * s.inv_optim_scale : in_m / s.optim_scale;
        const float v_un = pow2 ? in_v * s.inv_optim_scale : in_v / s.optim_scale;
        momentum = s.b1 * m_un + s.one_minus_b1 * scaled_grad;
        velocity = s.b2 * v_un + (s.one_minus_b2 * scaled_grad) * scaled_grad;
        out_m = momentum * s.optim_scale;
        out_v = velocity * s.optim_scale;
    } else {
        momentum = s.b1 * in_m + s.one_minus_b1 * scaled_grad;
        velocity = s.b2 * in_v + (s.one_minus_b2 * scaled_grad) * scaled_grad;
        out_m = momentum;
        out_v = velocity;
    }
    const float denom = (s.eps_mode == 0) ? sqrtf(velocity + s.eps) : sqrtf(velocity) + s.eps;
    const float update = momentum / denom + s.decay * in_p;
    out_p = in_p - s.step_size * update;
}

template <typename T>
__device__ __forceinline__ float load_scalar(gptr<const T> ptr) { return (float)*ptr; }
__device__ __forceinline__ void store_scalar(gptr<float> ptr, float x) { *ptr = x; }
__device__ __forceinline__ bool store_scalar(gptr<_Float16> ptr, float x, bool check) {
    const _Float16 h = (_Float16)x;
    *ptr = h;
    return check && ((__builtin_bit_cast(uint16_t, h) & 0x7c00u) == 0x7c00u);
}

// One element through the element-wise path (tails and misaligned tensors).
template <int MODE>
__device__ __forceinline__ bool step_element(const StepScalars& s, gptr<typename ModeTraits<MODE>::P> p,
                                             gptr<typename ModeTraits<MODE>::S> m, gptr<typename ModeTraits<MODE>::S> v,
                                             gptr<const typename ModeTraits<MODE>::G> g, gptr<_Float16> p_copy) {
    using T = ModeTraits<MODE>;
    float np, nm, nv;
    adam_update<T::kScaled>(s, load_scalar<typename T::P>(p), load_scalar<typename T::S>(m),
                            load_scalar<typename T::S>(v), load_scalar<typename T::G>(g), np, nm, nv);
    bool bad = false;
    if constexpr (sizeof(typename T::S) == 2) {
        bad |= store_scalar(m, nm, true);
        bad |= store_scalar(v, nv, true);
    } else {
        store_scalar(m, nm);
        store_scalar(v, nv);
    }
    if constexpr (sizeof(typename T::P) == 2) {
        store_scalar(p, np, false);
    } else {
        store_scalar(p, np);
        if constexpr (T::kCopy) store_scalar(p_copy, np, false);  // half(stored fp32 p): kernel.cu:129
    }
    return bad;
}

// kVec consecutive elements of every stream through registers.
template <int MODE, bool NT>
struct VectorStep {
    using T = ModeTraits<MODE>;
    static constexpr int kVec = T::kVec;
    Packet<typename T::P, kVec> rp;
    Packet<typename T::S, kVec> rm, rv;
    Packet<typename T::G, kVec> rg;

    __device__ __forceinline__ void load(gptr<const typename T::P> p, gptr<const typename T::S> m,
                                         gptr<const typename T::S> v, gptr<const typename T::G> g) {
        rp = load_packet<typename T::P, kVec, NT>(p);
        rm = load_packet<typename T::S, kVec, NT>(m);
        rv = load_packet<typename T::S, kVec, NT>(v);
        rg = load_packet<typename T::G, kVec, NT>(g);
    }
    __device__ __forceinline__ bool compute_store(const StepScalars& s, gptr<typename T::P> p, gptr<typename T::S> m,
                                                  gptr<typename T::S> v, gptr<_Float16> p_copy) {
        float fp[kVec], fm[kVec], fv[kVec], fg[kVec];
        unpack(rp, fp);
        unpack(rm, fm);
        unpack(rv, fv);
        unpack(rg, fg);
#pragma unroll
        for (int k = 0; k < kVec; ++k) adam_update<T::kScaled>(s, fp[k], fm[k], fv[k], fg[k], fp[k], fm[k], fv[k]);
        bool bad = false;
        Packet<typename T::S, kVec> om, ov;
        if constexpr (sizeof(typename T::S) == 2) {
            bad |= pack(fm, om);
            bad |= pack(fv, ov);
        } else {
            pack(fm, om);
            pack(fv, ov);
        }
        store_packet<typename T::S, kVec, NT>(m, om);
        store_packet<typename T::S, kVec, NT>(v, ov);
        Packet<typename T::P, kVec> op;
        pack(fp, op);
        store_packet<typename T::P, kVec, NT>(p, op);
        if constexpr (T::kCopy) {
            Packet<_Float16, kVec> oc;
            pack(fp, oc);
            store_packet<_Float16, kVec, NT>(p_copy, oc);
        }
        return bad;
    }
};

template <int MODE, int UNROLL, bool NT>
__global__ __launch_bounds__(kBlock) void fsadam_kernel(const TensorRow* __restrict__ table,
                                                        const uint32_t* __restrict__ chunk_prefix,
                                                        uint32_t n_tensors, uint32_t n_chunks, uint32_t chunk_elems,
                                                        StepScalars s, float* __restrict__ found_inf) {
    using T = ModeTraits<MODE>;
    constexpr int kVec = T::kVec;
    extern __shared__ uint32_t lds_prefix[];  // n_tensors + 1 entries, relative to this launch's first chunk

    const uint32_t first = chunk_prefix[0];
    for (uint32_t i = threadIdx.x; i <= n_tensors; i += kBlock) lds_prefix[i] = chunk_prefix[i] - first;
    __syncthreads();

    bool bad = false;
    for (uint32_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
        // last tensor t with lds_prefix[t] <= c  (tensors without elements have an empty range and are never hit)
        uint32_t lo = 0, hi = n_tensors;  // invariant: lds_prefix[lo] <= c < lds_prefix[hi]
        while (hi - lo > 1) {
            const uint32_t mid = (lo + hi) >> 1;
            if (lds_prefix[mid] <= c) lo = mid; else hi = mid;
        }
        const uint32_t t = __builtin_amdgcn_readfirstlane(lo);
        const uint32_t local_chunk = __builtin_amdgcn_readfirstlane(c - lds_prefix[lo]);
        const TensorRow row = table[t];
        const int64_t base = (int64_t)local_chunk * chunk_elems;
        const int64_t left = row.numel - base;
        const int n = (int)(left < (int64_t)chunk_elems ? left : (int64_t)chunk_elems);

        gptr<typename T::P> p = (gptr<typename T::P>)row.p + base;
        gptr<typename T::S> m = (gptr<typename T::S>)row.m + base;
        gptr<typename T::S> v = (gptr<typename T::S>)row.v + base;
        gptr<const typename T::G> g = (gptr<const typename T::G>)row.g + base;
        gptr<_Float16> pc = T::kCopy ? (gptr<_Float16>)row.p_copy + base : nullptr;

        if (row.vector_ok) {
            const int nvec = n / kVec;
            int i = threadIdx.x;
            for (; i + (UNROLL - 1) * kBlock < nvec; i += UNROLL * kBlock) {
                VectorStep<MODE, NT> st[UNROLL];
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const int64_t e = (int64_t)(i + u * kBlock) * kVec;
                    st[u].load(p + e, m + e, v + e, g + e);
                }
#pragma unroll
                for (int u = 0; u < UNROLL; ++u) {
                    const int64_t e = (int64_t)(i + u * kBlock) * kVec;
                    bad |= st[u].compute_store(s, p + e, m + e, v + e, T::kCopy ? pc + e : nullptr);
                }
            }
            for (; i < nvec; i += kBlock) {
                VectorStep<MODE, NT> st;
                const int64_t e = (int64_t)i * kVec;
                st.load(p + e, m + e, v + e, g + e);
                bad |= st.compute_store(s, p + e, m + e, v + e, T::kCopy ? pc + e : nullptr);
            }
            const int e = nvec * kVec + (int)threadIdx.x;  // fewer than kVec ragged elements at the end of a tensor
            if (e < n) bad |= step_element<MODE>(s, p + e, m + e, v + e, g + e, T::kCopy ? pc + e : nullptr);
        } else {
#pragma unroll 4
            for (int e = threadIdx.x; e < n; e += kBlock)
                bad |= step_element<MODE>(s, p + e, m + e, v + e, g + e, T::kCopy ? pc + e : nullptr);
        }
    }
    // Same-value store from every lane that saw a non-finite stored half (kernel.cu:103-105).
    if (T::kScaled && bad) *(gptr<float>)found_inf = 1.0f;
}

__global__ __launch_bounds__(kBlock) void fsadam_copy_kernel(f32x4* __restrict__ dst_, const f32x4* __restrict__ src_,
                                                             int64_t n_quads) {
    gptr<f32x4> dst = (gptr<f32x4>)dst_;
    gptr<const f32x4> src = (gptr<const f32x4>)src_;
    const int64_t stride = (int64_t)gridDim.x * kBlock;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < n_quads; i += stride)
        __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
}

// --------------------------------------------------------------------------------------------
// host side
// --------------------------------------------------------------------------------------------

thread_local std::string g_last_error;

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}
int fail_hip(hipError_t e, const char* what) {
    return fail(FSADAM_EHIP, std::string(what) + ": " + hipGetErrorString(e));
}
#define FS_HIP(call)                                       \
    do {                                                   \
        hipError_t e_ = (call);                            \
        if (e_ != hipSuccess) return fail_hip(e_, #call); \
    } while (0)

struct Options {
    int64_t chunk_elems = 16384;
    int64_t wg_per_cu = 8;
    int64_t nontemporal = 1;
    int64_t unroll = 2;
};
Options g_opt;
std::mutex g_mutex;        // guards g_opt
std::mutex g_cache_mutex;  // guards the fsadam_step table cache

bool valid_mode(int mode) { return mode >= FSADAM_FULL_PRECISION && mode <= FSADAM_PURE_FP16; }

int elem_size_p(int mode) { return (mode == FSADAM_FULL_PRECISION || mode == FSADAM_MIXED_PRECISION) ? 4 : 2; }

bool aligned16(const void* ptr) { return (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0; }

bool is_pow2_with_exact_reciprocal(float x, float* inv) {
    if (!(x > 0.0f) || !std::isfinite(x)) return false;
    int e;
    const float mant = std::frexp(x, &e);
    if (mant != 0.5f) return false;
    const float r = 1.0f / x;
    if (!std::isnormal(x) || !std::isnormal(r)) return false;
    *inv = r;
    return true;
}

int validate_rows(const FsAdamTensor* tensors, int64_t n, int mode) {
    if (!valid_mode(mode)) return fail(FSADAM_EINVAL, "unknown precision mode " + std::to_string(mode));
    if (n < 1) return fail(FSADAM_EINVAL, "tensor list is empty");  // multi_tensor_apply.cuh:51
    if (!tensors) return fail(FSADAM_EINVAL, "tensors is NULL");
    for (int64_t t = 0; t < n; ++t) {
        const FsAdamTensor& r = tensors[t];
        if (r.numel < 0) return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": negative numel");
        if (r.numel == 0) continue;
        if (!r.p || !r.m || !r.v || !r.g) return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": NULL p/m/v/g pointer");
        if (mode == FSADAM_MIXED_PRECISION && !r.p_copy)
            return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": MIXED_PRECISION needs p_copy");
        // element alignment: anything less cannot be a tensor of that dtype
        const uintptr_t pa = elem_size_p(mode) - 1, sa = (mode == FSADAM_PURE_FP16 ? 2 : 4) - 1,
                        ga = (mode == FSADAM_FULL_PRECISION ? 4 : 2) - 1;
        if ((reinterpret_cast<uintptr_t>(r.p) & pa) || (reinterpret_cast<uintptr_t>(r.m) & sa) ||
            (reinterpret_cast<uintptr_t>(r.v) & sa) || (reinterpret_cast<uintptr_t>(r.g) & ga) ||
            (mode == FSADAM_MIXED_PRECISION && (reinterpret_cast<uintptr_t>(r.p_copy) & 1)))
            return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": pointer not aligned to its element size");
    }
    return FSADAM_OK;
}

bool row_vector_ok(const FsAdamTensor& r, int mode) {
    return aligned16(r.p) && aligned16(r.m) && aligned16(r.v) && aligned16(r.g) &&
           (mode != FSADAM_MIXED_PRECISION || aligned16(r.p_copy));
}

int64_t chunks_of(int64_t numel, int64_t chunk_elems) { return (numel + chunk_elems - 1) / chunk_elems; }

}  // namespace

struct FsAdamPlan {
    int mode = 0;
    int device = -1;
    int cu_count = 0;
    Options opt;
    std::vector<FsAdamTensor> rows;  // what the device table was built from
    int64_t total_elems = 0, total_chunks = 0, n_vector = 0, n_scalar = 0, uploads = 0;
    // one device allocation: TensorRow[cap_tensors] then uint32_t[cap_tensors + 1]
    int64_t cap_tensors = 0;
    void* d_buf = nullptr;
    void* h_buf = nullptr;  // pinned staging of the same layout
    hipEvent_t last_use = nullptr;
    bool used = false;
    uint64_t lru = 0;  // fsadam_step cache bookkeeping

    TensorRow* d_rows() const { return static_cast<TensorRow*>(d_buf); }
    uint32_t* d_prefix() const { return reinterpret_cast<uint32_t*>(static_cast<char*>(d_buf) + cap_tensors * sizeof(TensorRow)); }
    TensorRow* h_rows() const { return static_cast<TensorRow*>(h_buf); }
    uint32_t* h_prefix() const { return reinterpret_cast<uint32_t*>(static_cast<char*>(h_buf) + cap_tensors * sizeof(TensorRow)); }
    size_t buf_bytes() const { return cap_tensors * sizeof(TensorRow) + (cap_tensors + 1) * sizeof(uint32_t); }
};

namespace {

int plan_release_buffers(FsAdamPlan* plan) {
    if (plan->used && plan->last_use) (void)hipEventSynchronize(plan->last_use);
    if (plan->d_buf) (void)hipFree(plan->d_buf);
    if (plan->h_buf) (void)hipHostFree(plan->h_buf);
    plan->d_buf = plan->h_buf = nullptr;
    plan->cap_tensors = 0;
    return FSADAM_OK;
}

template <int MODE>
int launch_mode(const FsAdamPlan* plan, const StepScalars& s, float* found_inf, hipStream_t stream) {
    const int64_t n = (int64_t)plan->rows.size();
    const uint32_t* hp = plan->h_prefix();
    for (int64_t t0 = 0; t0 < n; t0 += kWindow) {
        const int64_t nt = std::min<int64_t>(kWindow, n - t0);
        const uint32_t n_chunks = hp[t0 + nt] - hp[t0];
        if (n_chunks == 0) continue;
        const int64_t want = (int64_t)plan->cu_count * plan->opt.wg_per_cu;
        const uint32_t grid = (uint32_t)std::max<int64_t>(1, std::min<int64_t>(n_chunks, want));
        const size_t lds = (size_t)(nt + 1) * sizeof(uint32_t);
        const TensorRow* rows = plan->d_rows() + t0;
        const uint32_t* prefix = plan->d_prefix() + t0;
        const uint32_t chunk_elems = (uint32_t)plan->opt.chunk_elems;
#define FS_LAUNCH(U, NT)                                                                                    \
    hipLaunchKernelGGL((fsadam_kernel<MODE, U, NT>), dim3(grid), dim3(kBlock), lds, stream, rows, prefix, \
                       (uint32_t)nt, n_chunks, chunk_elems, s, found_inf)
        const bool nt_hint = plan->opt.nontemporal != 0;
        switch (plan->opt.unroll) {
            case 1: if (nt_hint) FS_LAUNCH(1, true); else FS_LAUNCH(1, false); break;
            case 4: if (nt_hint) FS_LAUNCH(4, true); else FS_LAUNCH(4, false); break;
            default: if (nt_hint) FS_LAUNCH(2, true); else FS_LAUNCH(2, false); break;
        }
#undef FS_LAUNCH
        FS_HIP(hipGetLastError());
    }
    return FSADAM_OK;
}

int plan_set_tensors(FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n, hipStream_t stream) {
    int rc = validate_rows(tensors, n, plan->mode);
    if (rc) return rc;
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (plan->device != dev) {
        if (plan->d_buf) plan_release_buffers(plan);
        plan->device = dev;
        FS_HIP(hipDeviceGetAttribute(&plan->cu_count, hipDeviceAttributeMultiprocessorCount, dev));
        if (plan->cu_count < 1) return fail(FSADAM_ENODEVICE, "device reports no compute units");
        if (!plan->last_use) FS_HIP(hipEventCreateWithFlags(&plan->last_use, hipEventDisableTiming));
    }
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        plan->opt = g_opt;
    }
    const int64_t chunk_elems = plan->opt.chunk_elems;
    uint64_t chunks = 0;
    for (int64_t t = 0; t < n; ++t) chunks += (uint64_t)chunks_of(tensors[t].numel, chunk_elems);
    if (chunks > 0xffffffffull) return fail(FSADAM_EINVAL, "tensor list needs more than 2^32 chunks; raise chunk_elems");

    // the previous table may still be read by a kernel in flight
    if (plan->used) FS_HIP(hipEventSynchronize(plan->last_use));
    if (n > plan->cap_tensors) {
        plan_release_buffers(plan);
        plan->cap_tensors = std::max<int64_t>(n, 16);
        if (hipMalloc(&plan->d_buf, plan->buf_bytes()) != hipSuccess) {
            plan->d_buf = nullptr; plan->cap_tensors = 0;
            return fail(FSADAM_ENOMEM, "hipMalloc of the tensor table failed");
        }
        if (hipHostMalloc(&plan->h_buf, plan->buf_bytes(), hipHostMallocDefault) != hipSuccess) {
            (void)hipFree(plan->d_buf);
            plan->d_buf = plan->h_buf = nullptr; plan->cap_tensors = 0;
            return fail(FSADAM_ENOMEM, "hipHostMalloc of the table staging buffer failed");
        }
    }
    TensorRow* hr = plan->h_rows();
    uint32_t* hp = plan->h_prefix();
    plan->total_elems = 0; plan->n_vector = 0; plan->n_scalar = 0;
    uint32_t run = 0;
    for (int64_t t = 0; t < n; ++t) {
        const FsAdamTensor& r = tensors[t];
        const bool vec = r.numel > 0 && row_vector_ok(r, plan->mode);
        hr[t] = TensorRow{r.p, r.m, r.v, r.g, r.p_copy, r.numel, vec ? 1u : 0u, 0u};
        hp[t] = run;
        run += (uint32_t)chunks_of(r.numel, chunk_elems);
        plan->total_elems += r.numel;
        if (r.numel > 0) (vec ? plan->n_vector : plan->n_scalar) += 1;
    }
    hp[n] = run;
    plan->total_chunks = run;
    plan->rows.assign(tensors, tensors + n);
    // rows and prefix are not adjacent when n < cap_tensors: two copies
    FS_HIP(hipMemcpyAsync(plan->d_rows(), hr, (size_t)n * sizeof(TensorRow), hipMemcpyHostToDevice, stream));
    FS_HIP(hipMemcpyAsync(plan->d_prefix(), hp, (size_t)(n + 1) * sizeof(uint32_t), hipMemcpyHostToDevice, stream));
    FS_HIP(hipEventRecord(plan->last_use, stream));
    plan->used = true;
    plan->uploads += 1;
    return FSADAM_OK;
}

int plan_step(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, float grad_scale, float optim_scale,
              float decay, int step, int eps_mode, int bias_correction, float* found_inf, hipStream_t stream) {
    if (plan->rows.empty() || !plan->d_buf) return fail(FSADAM_EINVAL, "plan has no tensors; call fsadam_plan_set_tensors first");
    if (eps_mode != FSADAM_EPS_INSIDE_SQRT && eps_mode != FSADAM_EPS_OUTSIDE_SQRT)
        return fail(FSADAM_EINVAL, "eps_mode must be 0 (inside sqrt) or 1 (outside)");
    if (plan->mode == FSADAM_PURE_FP16 && !found_inf) return fail(FSADAM_EINVAL, "PURE_FP16 needs a found_inf device pointer");
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (dev != plan->device) return fail(FSADAM_EINVAL, "plan belongs to device " + std::to_string(plan->device) + ", current device is " + std::to_string(dev));

    StepScalars s;
    s.b1 = beta1; s.b2 = beta2;
    s.one_minus_b1 = 1 - beta1;  // float subtraction as in the device code of the reference (kernel.cu:97,118)
    s.one_minus_b2 = 1 - beta2;
    s.eps = eps; s.decay = decay;
    s.step_size = fsadam_step_size(lr, beta1, beta2, step, bias_correction);
    s.grad_scale = grad_scale; s.optim_scale = optim_scale;
    s.inv_grad_scale = 0.f; s.inv_optim_scale = 0.f;
    s.eps_mode = eps_mode;
    s.flags = 0;
    if (is_pow2_with_exact_reciprocal(grad_scale, &s.inv_grad_scale)) s.flags |= kGradScalePow2;
    if (is_pow2_with_exact_reciprocal(optim_scale, &s.inv_optim_scale)) s.flags |= kOptimScalePow2;

    int rc;
    switch (plan->mode) {
        case FSADAM_FULL_PRECISION: rc = launch_mode<FSADAM_FULL_PRECISION>(plan, s, found_inf, stream); break;
        case FSADAM_MIXED_PRECISION: rc = launch_mode<FSADAM_MIXED_PRECISION>(plan, s, found_inf, stream); break;
        case FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION: rc = launch_mode<FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION>(plan, s, found_inf, stream); break;
        default: rc = launch_mode<FSADAM_PURE_FP16>(plan, s, found_inf, stream); break;
    }
    if (rc) return rc;
    FS_HIP(hipEventRecord(plan->last_use, stream));
    return FSADAM_OK;
}

// fsadam_step's table cache
constexpr size_t kCacheWays = 8;
std::vector<FsAdamPlan*> g_cache;
uint64_t g_tick = 0;

bool same_rows(const FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n) {
    if ((int64_t)plan->rows.size() != n) return false;
    for (int64_t t = 0; t < n; ++t) {
        const FsAdamTensor &a = plan->rows[t], &b = tensors[t];
        if (a.p != b.p || a.m != b.m || a.v != b.v || a.g != b.g || a.p_copy != b.p_copy || a.numel != b.numel) return false;
    }
    return true;
}

}  // namespace

extern "C" {

int fsadam_version(void) { return FSADAM_ABI_VERSION; }

const char* fsadam_last_error(void) { return g_last_error.c_str(); }

float fsadam_step_size(float lr, float beta1, float beta2, int step, int bias_correction) {
    if (bias_correction == 1) {
        // std::pow(float, int) is evaluated in double; the difference is narrowed to float (kernel.cu:156-157)
        const float bc1 = (float)(1.0 - std::pow((double)beta1, (double)step));
        const float bc2 = (float)(1.0 - std::pow((double)beta2, (double)step));
        const float root = std::sqrt(bc2);
        const float num = lr * root;
        return num / bc1;
    }
    return lr;
}

int fsadam_set_option(const char* name, int64_t value) {
    if (!name) return fail(FSADAM_EINVAL, "option name is NULL");
    std::lock_guard<std::mutex> lock(g_mutex);
    const std::string k(name);
    if (k == "chunk_elems") {
        if (value < kChunkQuantum || value % kChunkQuantum || value > (1 << 30)) return fail(FSADAM_EINVAL, "chunk_elems must be a multiple of 2048 in [2048, 2^30]");
        g_opt.chunk_elems = value;
    } else if (k == "wg_per_cu") {
        if (value < 1 || value > (1 << 24)) return fail(FSADAM_EINVAL, "wg_per_cu must be in [1, 2^24]");
        g_opt.wg_per_cu = value;
    } else if (k == "nontemporal") {
        if (value != 0 && value != 1) return fail(FSADAM_EINVAL, "nontemporal must be 0 or 1");
        g_opt.nontemporal = value;
    } else if (k == "unroll") {
        if (value != 1 && value != 2 && value != 4) return fail(FSADAM_EINVAL, "unroll must be 1, 2 or 4");
        g_opt.unroll = value;
    } else {
        return fail(FSADAM_EINVAL, "unknown option '" + k + "'");
    }
    return FSADAM_OK;
}

int fsadam_get_option(const char* name, int64_t* value) {
    if (!name || !value) return fail(FSADAM_EINVAL, "NULL argument");
    std::lock_guard<std::mutex> lock(g_mutex);
    const std::string k(name);
    if (k == "chunk_elems") *value = g_opt.chunk_elems;
    else if (k == "wg_per_cu") *value = g_opt.wg_per_cu;
    else if (k == "nontemporal") *value = g_opt.nontemporal;
    else if (k == "unroll") *value = g_opt.unroll;
    else return fail(FSADAM_EINVAL, "unknown option '" + k + "'");
    return FSADAM_OK;
}

int fsadam_layout(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, int64_t chunk_elems,
                  uint64_t* chunk_prefix, uint8_t* vector_ok) {
    int rc = validate_rows(tensors, n_tensors, precision_mode);
    if (rc) return rc;
    if (chunk_elems < kChunkQuantum || chunk_elems % kChunkQuantum) return fail(FSADAM_EINVAL, "chunk_elems must be a positive multiple of 2048");
    if (!chunk_prefix || !vector_ok) return fail(FSADAM_EINVAL, "NULL output");
    uint64_t run = 0;
    for (int64_t t = 0; t < n_tensors; ++t) {
        chunk_prefix[t] = run;
        run += (uint64_t)chunks_of(tensors[t].numel, chunk_elems);
        vector_ok[t] = (tensors[t].numel > 0 && row_vector_ok(tensors[t], precision_mode)) ? 1 : 0;
    }
    chunk_prefix[n_tensors] = run;
    return FSADAM_OK;
}

int fsadam_plan_create(int precision_mode, FsAdamPlan** out) {
    if (!out) return fail(FSADAM_EINVAL, "out is NULL");
    if (!valid_mode(precision_mode)) return fail(FSADAM_EINVAL, "unknown precision mode " + std::to_string(precision_mode));
    FsAdamPlan* plan = new (std::nothrow) FsAdamPlan();
    if (!plan) return fail(FSADAM_ENOMEM, "out of host memory");
    plan->mode = precision_mode;
    *out = plan;
    return FSADAM_OK;
}

int fsadam_plan_set_tensors(FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n_tensors, void* hip_stream) {
    if (!plan) return fail(FSADAM_EINVAL, "plan is NULL");
    return plan_set_tensors(plan, tensors, n_tensors, static_cast<hipStream_t>(hip_stream));
}

int fsadam_plan_step(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, float grad_scale,
                     float optim_scale, float decay, int step, int eps_mode, int bias_correction,
                     float* found_inf_dev, void* hip_stream) {
    if (!plan) return fail(FSADAM_EINVAL, "plan is NULL");
    return plan_step(plan, lr, beta1, beta2, eps, grad_scale, optim_scale, decay, step, eps_mode, bias_correction,
                     found_inf_dev, static_cast<hipStream_t>(hip_stream));
}

int fsadam_plan_info(const FsAdamPlan* plan, FsAdamPlanInfo* out) {
    if (!plan || !out) return fail(FSADAM_EINVAL, "NULL argument");
    std::memset(out, 0, sizeof(*out));
    out->mode = plan->mode;
    out->device = plan->device;
    out->n_tensors = (int64_t)plan->rows.size();
    out->total_elems = plan->total_elems;
    out->total_chunks = plan->total_chunks;
    out->chunk_elems = plan->opt.chunk_elems;
    out->n_vector_tensors = plan->n_vector;
    out->n_scalar_tensors = plan->n_scalar;
    out->n_launches = 0;
    out->grid = 0;
    if (plan->h_buf) {
        const int64_t n = (int64_t)plan->rows.size();
        const uint32_t* hp = plan->h_prefix();
        for (int64_t t0 = 0; t0 < n; t0 += kWindow) {
            const int64_t nt = std::min<int64_t>(kWindow, n - t0);
            const uint32_t n_chunks = hp[t0 + nt] - hp[t0];
            if (!n_chunks) continue;
            if (out->n_launches == 0) out->grid = std::max<int64_t>(1, std::min<int64_t>(n_chunks, (int64_t)plan->cu_count * plan->opt.wg_per_cu));
            out->n_launches += 1;
        }
    }
    out->block = kBlock;
    out->uploads = plan->uploads;
    return FSADAM_OK;
}

int fsadam_plan_destroy(FsAdamPlan* plan) {
    if (!plan) return FSADAM_OK;
    plan_release_buffers(plan);
    if (plan->last_use) (void)hipEventDestroy(plan->last_use);
    delete plan;
    return FSADAM_OK;
}

int fsadam_step(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, float lr, float beta1,
                float beta2, float eps, float grad_scale, float optim_scale, float decay, int step,
                int eps_mode, int bias_correction, float* found_inf_dev, void* hip_stream) {
    int rc = validate_rows(tensors, n_tensors, precision_mode);
    if (rc) return rc;
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    FsAdamPlan* hit = nullptr;
    FsAdamPlan* victim = nullptr;
    for (FsAdamPlan* c : g_cache) {
        if (c->device == dev && c->mode == precision_mode && same_rows(c, tensors, n_tensors)) { hit = c; break; }
        if (c->mode == precision_mode && (c->device == dev || c->device < 0) && (!victim || c->lru < victim->lru)) victim = c;
    }
    if (!hit) {
        if (g_cache.size() < kCacheWays || !victim) {
            FsAdamPlan* fresh = nullptr;
            rc = fsadam_plan_create(precision_mode, &fresh);
            if (rc) return rc;
            if (g_cache.size() >= kCacheWays) {  // every way holds another mode/device: drop the oldest
                size_t oldest = 0;
                for (size_t i = 1; i < g_cache.size(); ++i) if (g_cache[i]->lru < g_cache[oldest]->lru) oldest = i;
                fsadam_plan_destroy(g_cache[oldest]);
                g_cache[oldest] = fresh;
            } else {
                g_cache.push_back(fresh);
            }
            victim = fresh;
        }
        rc = plan_set_tensors(victim, tensors, n_tensors, stream);
        if (rc) { victim->rows.clear(); return rc; }
        hit = victim;
    }
    hit->lru = ++g_tick;
    return plan_step(hit, lr, beta1, beta2, eps, grad_scale, optim_scale, decay, step, eps_mode, bias_correction,
                     found_inf_dev, stream);
}

int fsadam_clear_cache(void) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (FsAdamPlan* c : g_cache) fsadam_plan_destroy(c);
    g_cache.clear();
    return FSADAM_OK;
}

int fsadam_calib_copy(void* dst, const void* src, int64_t nbytes, void* hip_stream) {
    if (!dst || !src || nbytes < 0 || (nbytes & 15) || !aligned16(dst) || !aligned16(src))
        return fail(FSADAM_EINVAL, "calib copy needs 16-byte aligned pointers and a multiple of 16 bytes");
    if (nbytes == 0) return FSADAM_OK;
    int dev = -1, cus = 0;
    FS_HIP(hipGetDevice(&dev));
    FS_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int64_t quads = nbytes / 16;
    const int64_t grid = std::max<int64_t>(1, std::min<int64_t>((quads + kBlock - 1) / kBlock, (int64_t)cus * 8));
    hipLaunchKernelGGL(fsadam_copy_kernel, dim3((uint32_t)grid), dim3(kBlock), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<f32x4*>(dst), static_cast<const f32x4*>(src), quads);
    FS_HIP(hipGetLastError());
    return FSADAM_OK;
}

}  // extern "C"
