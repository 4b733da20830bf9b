// Device code of the Adam step: vector and element-wise tile bodies and the kernel fsadam_tiles.
// Reference: fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:21-135 (AdamFunctor) and the
// per-block prologue of fairscale/clib/fused_adam_cuda/multi_tensor_apply.cuh:28-38.
// Included by fsadam.hip only (one translation unit).
#pragma once

#include <hip/hip_runtime.h>

#include "fsadam_common.h"

namespace {

// --------------------------------------------------------------------------------------------
// device code
// --------------------------------------------------------------------------------------------

template <typename T, int E>
struct VecOf {
    typedef T type __attribute__((ext_vector_type(E)));
    // The same vector as it lies in memory: promised to be aligned like one element only.  Global
    // memory instructions of this target take any address (code for amdhsa is generated under that
    // assumption throughout), so the access is still one dwordx2/dwordx4 instruction; a stream
    // that starts at an odd element (a view into a flat buffer) costs a cache line more per wave,
    // not an element-by-element loop.
    typedef type in_memory __attribute__((aligned(sizeof(T))));
};

// E consecutive elements of one stream, one instruction: loads non-temporal, stores written through.
template <typename T, int E>
__device__ __forceinline__ typename VecOf<T, E>::type load_vec(gptr<const T> ptr) {
    using V = typename VecOf<T, E>::in_memory;
    return __builtin_nontemporal_load(reinterpret_cast<gptr<const V>>(ptr));
}
template <typename T, int E>
__device__ __forceinline__ void store_vec(gptr<T> ptr, typename VecOf<T, E>::type value) {
    store_through((gptr<void>)ptr, value);
}

// Two packed halves in one 32-bit word: non-zero when either is +-inf or NaN (exponent field all
// ones).  Adding 0x0400 to an all-ones exponent field carries into the sign position; any smaller
// field does not, and the low half cannot carry into the high one.  Whole words, three integer
// operations per two halves.  (A per-element form, __builtin_bit_cast(uint16_t, h[e]) on the elements
// of a half vector, silently tested element 0 eight times: this compiler's bit_cast of a vector
// ELEMENT always reads element 0.  Bit-cast whole vectors, or copy the element to a scalar first.)
__device__ __forceinline__ uint32_t nonfinite_halves(uint32_t w) {
    return ((w & 0x7c007c00u) + 0x04000400u) & 0x80008000u;
}

template <int E>
__device__ __forceinline__ uint32_t nonfinite_in(typename VecOf<_Float16, E>::type h) {
    static_assert(E == 4 || E == 8, "whole 32-bit words only");
    typedef uint32_t words_t __attribute__((ext_vector_type(E / 2)));
    const words_t w = __builtin_bit_cast(words_t, h);
    uint32_t bad = 0;
#pragma unroll
    for (int k = 0; k < E / 2; ++k) bad |= nonfinite_halves(w[k]);
    return bad;
}

// A float that is about to be narrowed to half passes through here first.  The compiler otherwise
// merges "multiply, then convert" into one v_fma_mixlo_f16, which rounds the exact product once;
// the reference (and the oracle) round to float32 first and to half afterwards, and the two differ
// when the float32 result lands exactly between two halves.  No instruction is emitted.
__device__ __forceinline__ float as_float32(float x) {
    asm("" : "+v"(x));
    return x;
}

// The update for one element, all in fp32 registers.
//   unscaled state: fused_adam_cuda_kernel.cu:115-130     scaled (fp16) state: :94-114
// out_m/out_v are what gets STORED (already multiplied by optim_scale when kScaled).
template <bool kScaled, int EPS_MODE, bool FAST_SCALES>
__device__ __forceinline__ void adam_update(const StepScalars& s, float in_p, float in_m, float in_v, float in_g,
                                            float& out_p, float& out_m, float& out_v) {
    const float scaled_grad = FAST_SCALES ? in_g * s.inv_grad_scale : in_g / s.grad_scale;
    float momentum, velocity;
    if (kScaled) {
        const float m_un = FAST_SCALES ? in_m * s.inv_optim_scale : in_m / s.optim_scale;
        const float v_un = FAST_SCALES ? in_v * s.inv_optim_scale : in_v / s.optim_scale;
        momentum = s.b1 * m_un + s.one_minus_b1 * scaled_grad;
        velocity = s.b2 * v_un + (s.one_minus_b2 * scaled_grad) * scaled_grad;
        out_m = as_float32(momentum * s.optim_scale);
        out_v = as_float32(velocity * s.optim_scale);
    } else {
        momentum = s.b1 * in_m + s.one_minus_b1 * scaled_grad;
        velocity = s.b2 * in_v + (s.one_minus_b2 * scaled_grad) * scaled_grad;
        out_m = momentum;
        out_v = velocity;
    }
    const float denom = (EPS_MODE == 0) ? sqrtf(velocity + s.eps) : sqrtf(velocity) + s.eps;
    const float update = momentum / denom + s.decay * in_p;
    out_p = as_float32(in_p - s.step_size * update);
}

// A full tile: GROUPS x (one vector per stream per lane), everything loaded before the
// first use.  Group k of the tile covers BLOCK*E consecutive elements, lane i the E elements at
// k*BLOCK*E + i*E, so each instruction of a wave touches one contiguous span.
template <int MODE, int BLOCK, int GROUPS, int EPS_MODE, bool FAST_SCALES>
__device__ __forceinline__ uint32_t tile_vector(const ChunkDesc& d, uint32_t off, const StepScalars& s) {
    using T = ModeTraits<MODE>;
    using P = typename T::P; using G = typename T::G; using S = typename T::S;
    constexpr int E = T::kElems;
    const uint32_t first = off + threadIdx.x * E;
    gptr<P> p = (gptr<P>)d.p + first;
    gptr<S> m = (gptr<S>)d.m + first;
    gptr<S> v = (gptr<S>)d.v + first;
    gptr<const G> g = (gptr<const G>)d.g + first;

    typename VecOf<P, E>::type rp[GROUPS];
    typename VecOf<S, E>::type rm[GROUPS], rv[GROUPS];
    typename VecOf<G, E>::type rg[GROUPS];
#pragma unroll
    for (int k = 0; k < GROUPS; ++k) {
        rp[k] = load_vec<P, E>(p + k * BLOCK * E);
        rm[k] = load_vec<S, E>(m + k * BLOCK * E);
        rv[k] = load_vec<S, E>(v + k * BLOCK * E);
        rg[k] = load_vec<G, E>(g + k * BLOCK * E);
    }
    uint32_t bad = 0;
#pragma unroll
    for (int k = 0; k < GROUPS; ++k) {
        typename VecOf<P, E>::type op;
        typename VecOf<S, E>::type om, ov;
        typename VecOf<_Float16, E>::type oc;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            float np, nm, nv;
            adam_update<T::kScaled, EPS_MODE, FAST_SCALES>(s, (float)rp[k][e], (float)rm[k][e], (float)rv[k][e],
                                                           (float)rg[k][e], np, nm, nv);
            op[e] = (P)np;  // round to nearest even when P is half
            om[e] = (S)nm;
            ov[e] = (S)nv;
            if constexpr (T::kCopy) oc[e] = (_Float16)np;  // half(stored fp32 p): kernel.cu:129
        }
        if constexpr (T::kScaled) bad |= nonfinite_in<E>(om) | nonfinite_in<E>(ov);
        store_vec<S, E>(m + k * BLOCK * E, om);
        store_vec<S, E>(v + k * BLOCK * E, ov);
        store_vec<P, E>(p + k * BLOCK * E, op);
        if constexpr (T::kCopy) store_vec<_Float16, E>((gptr<_Float16>)d.p_copy + first + k * BLOCK * E, oc);
    }
    return bad;
}

// Ragged tile (the end of a tensor): one element per lane per pass, same arithmetic.
template <int MODE, int BLOCK, int EPS_MODE, bool FAST_SCALES>
__device__ __forceinline__ uint32_t tile_elementwise(const ChunkDesc& d, uint32_t off, uint32_t count, const StepScalars& s) {
    using T = ModeTraits<MODE>;
    using P = typename T::P; using G = typename T::G; using S = typename T::S;
    gptr<P> p = (gptr<P>)d.p + off;
    gptr<S> m = (gptr<S>)d.m + off;
    gptr<S> v = (gptr<S>)d.v + off;
    gptr<const G> g = (gptr<const G>)d.g + off;
    gptr<_Float16> pc = T::kCopy ? (gptr<_Float16>)d.p_copy + off : nullptr;
    uint32_t bad = 0;
    for (uint32_t e = threadIdx.x; e < count; e += BLOCK) {
        float np, nm, nv;
        adam_update<T::kScaled, EPS_MODE, FAST_SCALES>(s, (float)p[e], (float)m[e], (float)v[e], (float)g[e], np, nm, nv);
        const S sm = (S)nm, sv = (S)nv;
        m[e] = sm;
        v[e] = sv;
        if constexpr (T::kScaled)
            bad |= nonfinite_halves((uint32_t)__builtin_bit_cast(uint16_t, sm) | ((uint32_t)__builtin_bit_cast(uint16_t, sv) << 16));
        p[e] = (P)np;
        if constexpr (T::kCopy) pc[e] = (_Float16)np;
    }
    return bad;
}

template <int MODE, int BLOCK, int GROUPS, int EPS_MODE, bool FAST_SCALES>
__device__ __forceinline__ uint32_t tile_any(const ChunkDesc& d, uint32_t off, const StepScalars& s) {
    constexpr uint32_t kTile = BLOCK * ModeTraits<MODE>::kElems * GROUPS;
    const uint32_t left = d.n - off;
    if (left >= kTile) return tile_vector<MODE, BLOCK, GROUPS, EPS_MODE, FAST_SCALES>(d, off, s);
    return tile_elementwise<MODE, BLOCK, EPS_MODE, FAST_SCALES>(d, off, left, s);
}

// One workgroup = one tile, which finds its descriptor through `map` (large tensors, middle-sized
// ones, then one descriptor per tile).  Tiles are taken in the order the hardware hands out workgroups:
// regrouping them so that each XCD (each L2) works on a contiguous range of its own was measured 3-6 %
// slower (nothing is read twice, so an L2 has nothing to keep, and the plain order spreads over the
// memory channels better).
template <int MODE, int BLOCK, int GROUPS>
__global__ __launch_bounds__(BLOCK) void fsadam_tiles(const ChunkDesc* __restrict__ table, TileMap map, StepScalars s,
                                                      float* __restrict__ found_inf) {
    constexpr uint32_t kTile = BLOCK * ModeTraits<MODE>::kElems * GROUPS;
    const uint32_t block = blockIdx.x;
    uint32_t chunk, off;
    locate_tile(map, block, kTile, chunk, off);
    // The whole 64-byte descriptor in ONE scalar load (uniform address, constant address space), before
    // anything is tested: reading the count first and the pointers afterwards would put two memory
    // latencies in front of the first data load.
    typedef uint32_t desc_words_t __attribute__((ext_vector_type(16)));
    const desc_words_t raw = *reinterpret_cast<const __attribute__((address_space(4))) desc_words_t*>(
        (const __attribute__((address_space(4))) ChunkDesc*)table + chunk);
    const ChunkDesc d = __builtin_bit_cast(ChunkDesc, raw);
    // A gradient scale that lives on the device (a clip factor or a loss scale computed there): one more
    // scalar load at a uniform address, issued next to the descriptor's.  The host has already switched
    // to true division (fast_scales = 0), which gives the bits of a host-side scale of the same value.
    if (s.grad_scale_dev) s.grad_scale = *(const __attribute__((address_space(4))) float*)s.grad_scale_dev;
    if (off >= d.n) return;  // tile past the end of its tensor (shared descriptors only)

    uint32_t bad;
    if (s.eps_mode == 0) {
        bad = s.fast_scales ? tile_any<MODE, BLOCK, GROUPS, 0, true>(d, off, s) : tile_any<MODE, BLOCK, GROUPS, 0, false>(d, off, s);
    } else {
        bad = s.fast_scales ? tile_any<MODE, BLOCK, GROUPS, 1, true>(d, off, s) : tile_any<MODE, BLOCK, GROUPS, 1, false>(d, off, s);
    }
    // Same-value store from every lane that stored a non-finite fp16 m or v (kernel.cu:103-105).
    if (ModeTraits<MODE>::kScaled && bad != 0) *(gptr<float>)found_inf = 1.0f;
}

// m = v = 0 over every tile of a step's table (same layout, same tile size): what follows an overflow of the fp16
// state (fairscale/optim/adam.py:285-288) in one launch, instead of a foreach over hundreds of tensors.
template <int MODE, int BLOCK>
__global__ __launch_bounds__(BLOCK) void fsadam_zero_state(const ChunkDesc* __restrict__ table, TileMap map) {
    using S = typename ModeTraits<MODE>::S;
    constexpr int E = ModeTraits<MODE>::kElems;
    constexpr uint32_t kTile = BLOCK * E;
    uint32_t chunk, off;
    locate_tile(map, blockIdx.x, kTile, chunk, off);
    typedef uint32_t desc_words_t __attribute__((ext_vector_type(16)));
    const desc_words_t raw = *reinterpret_cast<const __attribute__((address_space(4))) desc_words_t*>(
        (const __attribute__((address_space(4))) ChunkDesc*)table + chunk);
    const ChunkDesc d = __builtin_bit_cast(ChunkDesc, raw);
    if (off >= d.n) return;
    const uint32_t left = d.n - off;
    gptr<S> m = (gptr<S>)d.m + off;
    gptr<S> v = (gptr<S>)d.v + off;
    if (left >= kTile) {
        typename VecOf<S, E>::type zero = {};
        store_vec<S, E>(m + threadIdx.x * E, zero);
        store_vec<S, E>(v + threadIdx.x * E, zero);
    } else {
        for (uint32_t e = threadIdx.x; e < left; e += BLOCK) {
            m[e] = (S)0;
            v[e] = (S)0;
        }
    }
}

}  // namespace
