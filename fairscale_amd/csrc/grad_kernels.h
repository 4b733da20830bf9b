// Device code of the pre-step gradient pass (fsadam_grad_tiles, its two reduction kernels).
// Included by fsadam.hip only (one translation unit).
#pragma once

#include <hip/hip_runtime.h>

#include "fsadam_common.h"
#include "adam_kernels.h"

namespace {

// --------------------------------------------------------------------------------------------
// gradient pass: non-finite check + unscale + sum of squares + max |g| in ONE read of the gradients
// (what torch._amp_foreach_non_finite_check_and_unscale_, called from
// fairscale/optim/grad_scaler.py:211-215, and calc_grad_norm, fairscale/internal/params.py:59-76,
// do in two or more passes)
// --------------------------------------------------------------------------------------------

template <typename T>
struct GradTraits;
typedef uint32_t grad_words_t __attribute__((ext_vector_type(4)));
// 16 bytes of gradients as they lie in memory: aligned like one element only (see VecOf::in_memory)
template <>
struct GradTraits<float> {
    static constexpr int kElems = 4;
    typedef grad_words_t in_memory __attribute__((aligned(4)));
};
template <>
struct GradTraits<_Float16> {
    static constexpr int kElems = 8;
    typedef grad_words_t in_memory __attribute__((aligned(2)));
};

// Magnitudes are compared as integers: with the sign bit cleared, IEEE bit patterns order like the
// values, +inf is the largest finite-exponent pattern and every NaN is larger still.  One unsigned
// maximum therefore gives the max norm (a NaN wins, as in torch's abs().max()) and, taken over the
// incoming values, the overflow check (maximum >= the pattern of +inf) -- no floating compare, no
// per-element branch.  For halves two magnitudes travel in one 32-bit word (packed u16 maximum).
struct GradPartial {  // one per workgroup, written unconditionally
    double sum_squares;
    uint32_t stored_max;    // largest magnitude pattern of the values unscaling stores
    uint32_t incoming_max;  // largest magnitude pattern of the gradients as read
};

typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t max_u16x2(uint32_t a, uint32_t b) {
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}

// How the stored value r is formed from g: as is; by a packed half multiply (exact product, one
// rounding: the same bits as float(g) * inv_scale rounded to half whenever inv_scale is itself a
// half); or through float.
enum : int { kGradUnit = 0, kGradHalfScale = 1, kGradFloatScale = 2 };

// Only the largest incoming magnitude is tracked per element.  The largest STORED magnitude follows
// from it: g -> dtype(g * inv_scale) is a multiplication by a constant followed by roundings, all
// monotone in |g|, so the maximum of the results is the result of the maximum (NaN stays NaN, an
// overflow stays inf).  It is formed once per wave after the reduction.
struct GradAcc {
    float sum = 0.f;
    uint32_t incoming_max = 0;
};

// two halves in one word
template <int HOW>
__device__ __forceinline__ uint32_t grad_word(uint32_t w, float inv_scale, f16x2 inv_half, GradAcc& acc) {
    acc.incoming_max = max_u16x2(acc.incoming_max, w & 0x7fff7fffu);
    f16x2 r = __builtin_bit_cast(f16x2, w);
    if (HOW == kGradHalfScale) {
        r = r * inv_half;
    } else if (HOW == kGradFloatScale) {
        r[0] = (_Float16)as_float32((float)r[0] * inv_scale);
        r[1] = (_Float16)as_float32((float)r[1] * inv_scale);
    }
    const uint32_t out = __builtin_bit_cast(uint32_t, r);
    // fused multiply-adds with half operands widened on the fly (v_fma_mix_f32): the product of two
    // halves is exact in fp32, subnormal halves included
    acc.sum = __builtin_fmaf((float)r[0], (float)r[0], acc.sum);
    acc.sum = __builtin_fmaf((float)r[1], (float)r[1], acc.sum);
    return out;
}

// one half on its own (ragged tiles); the two scaled forms give the same bits.  Not grad_word on a word padded with a
// zero: under an infinite factor the padding would turn into 0 * inf = NaN and spoil the sum.
__device__ __forceinline__ _Float16 grad_scalar(_Float16 g, int how, float inv_scale, GradAcc& acc) {
    acc.incoming_max = max_u16x2(acc.incoming_max, (uint32_t)__builtin_bit_cast(uint16_t, g) & 0x7fffu);
    const _Float16 r = how == kGradUnit ? g : (_Float16)as_float32((float)g * inv_scale);
    acc.sum = __builtin_fmaf((float)r, (float)r, acc.sum);
    return r;
}

template <int HOW>
__device__ __forceinline__ float grad_float(float g, float inv_scale, GradAcc& acc) {
    const uint32_t mag = __builtin_bit_cast(uint32_t, g) & 0x7fffffffu;
    acc.incoming_max = mag > acc.incoming_max ? mag : acc.incoming_max;
    const float r = (HOW == kGradUnit) ? g : g * inv_scale;
    acc.sum += r * r;
    return r;
}

__device__ __forceinline__ float grad_scalar(float g, int how, float inv_scale, GradAcc& acc) {
    return how == kGradUnit ? grad_float<kGradUnit>(g, inv_scale, acc) : grad_float<kGradFloatScale>(g, inv_scale, acc);
}

// One wave's tile: BLOCK = 64 lanes, `lane` this thread's position in it.
template <typename T, int BLOCK, int ITEMS, int HOW, bool WRITE>
__device__ __forceinline__ void grad_tile(const ChunkDesc& d, uint32_t off, uint32_t lane, float inv_scale, GradAcc& acc) {
    constexpr int E = GradTraits<T>::kElems;
    constexpr uint32_t kTile = BLOCK * E * ITEMS;
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    using u32x4_in_memory = typename GradTraits<T>::in_memory;
    const uint32_t left = d.n - off;
    gptr<T> g = (gptr<T>)const_cast<void*>(d.g) + off;
    if (left >= kTile) {
        u32x4 raw[ITEMS];
#pragma unroll
        for (int k = 0; k < ITEMS; ++k)
            raw[k] = __builtin_nontemporal_load(reinterpret_cast<gptr<const u32x4_in_memory>>(g + (k * BLOCK + lane) * E));
        const f16x2 inv_half = {(_Float16)inv_scale, (_Float16)inv_scale};
#pragma unroll
        for (int k = 0; k < ITEMS; ++k) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // NB: copy the element out before __builtin_bit_cast: applied directly to a vector
                // element (bit_cast(T, v[e])) this compiler reads element 0 whatever e is.
                const uint32_t word = raw[k][e];
                if constexpr (sizeof(T) == 2) raw[k][e] = grad_word<HOW>(word, inv_scale, inv_half, acc);
                else raw[k][e] = __builtin_bit_cast(uint32_t, grad_float<HOW>(__builtin_bit_cast(float, word), inv_scale, acc));
            }
            if (WRITE && HOW != kGradUnit)
                store_through((gptr<void>)(g + (k * BLOCK + lane) * E), raw[k]);
        }
    } else {
        for (uint32_t e = lane; e < left; e += BLOCK) {
            const T r = grad_scalar(g[e], HOW, inv_scale, acc);
            if (WRITE && HOW != kGradUnit) g[e] = r;
        }
    }
}

// One wave = one tile of 64 x ITEMS 16-byte vectors, found through the table like the tiles of the
// Adam step.  A workgroup is WAVES consecutive tiles and writes ONE partial of 16 bytes.  Those small
// stores are what a pass over the gradients pays for besides its stream: written through one by one
// (400 000 to 800 000 stores of a quarter of a 64-byte memory word each) they cost a pass that only reads
// 5-8 % and a pass that writes back 2.5 %.  They are therefore ordinary cached stores, and workgroup b
// writes slot (b mod 8) * per_xcd + b / 8: the hardware deals consecutive workgroups out to the eight XCDs
// in turn, each XCD has an L2 of its own, so the eight partials that make up one 128-byte line all come
// from the same L2, a few workgroups apart in time, and leave it as one full line.  (Nothing depends on
// which XCD a workgroup really runs on: the slot is a function of the workgroup's number alone, and the
// reduction reads the slots in a fixed order.)  `n_tiles`: tiles really there (the last workgroup may
// have fewer than WAVES); `per_xcd`: ceil(workgroups / 8).
template <typename T, int WAVES, int ITEMS>
__global__ __launch_bounds__(64 * WAVES) void fsadam_grad_tiles(const ChunkDesc* __restrict__ table, TileMap map, uint32_t n_tiles, float inv_scale_value,
                                                                const float* __restrict__ inv_scale_dev, int write_back,
                                                                GradPartial* __restrict__ partials, uint32_t per_xcd) {
    constexpr int BLOCK = 64;
    constexpr uint32_t kTile = BLOCK * GradTraits<T>::kElems * ITEMS;
    // the wave's number within the workgroup is the same for all its lanes: say so, and the tile's
    // descriptor stays a scalar load
    const uint32_t wave = WAVES == 1 ? 0u : (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t lane = WAVES == 1 ? threadIdx.x : (threadIdx.x & 63u);
    const uint32_t block = blockIdx.x * WAVES + wave;
    // the scale may live on the device (a loss scaler keeps it there): uniform address, scalar load
    const float inv_scale = inv_scale_dev ? *(const __attribute__((address_space(4))) float*)inv_scale_dev : inv_scale_value;
    const bool half_scale = sizeof(T) == 2 && (float)(_Float16)inv_scale == inv_scale;

    GradAcc acc;
    bool any = false;  // uniform within the wave
    if (block < n_tiles) {
        uint32_t chunk, off;
        locate_tile(map, block, kTile, chunk, off);
        typedef uint32_t desc_words_t __attribute__((ext_vector_type(16)));
        const desc_words_t raw = *reinterpret_cast<const __attribute__((address_space(4))) desc_words_t*>(
            (const __attribute__((address_space(4))) ChunkDesc*)table + chunk);
        const ChunkDesc d = __builtin_bit_cast(ChunkDesc, raw);
        any = off < d.n;
        if (any) {
            if (inv_scale == 1.0f) {
                grad_tile<T, BLOCK, ITEMS, kGradUnit, false>(d, off, lane, inv_scale, acc);
            } else if (half_scale) {
                if (write_back) grad_tile<T, BLOCK, ITEMS, kGradHalfScale, true>(d, off, lane, inv_scale, acc);
                else grad_tile<T, BLOCK, ITEMS, kGradHalfScale, false>(d, off, lane, inv_scale, acc);
            } else {
                if (write_back) grad_tile<T, BLOCK, ITEMS, kGradFloatScale, true>(d, off, lane, inv_scale, acc);
                else grad_tile<T, BLOCK, ITEMS, kGradFloatScale, false>(d, off, lane, inv_scale, acc);
            }
        }
    }
    if (sizeof(T) == 2)  // unpack the two 16-bit maxima
        acc.incoming_max = (acc.incoming_max & 0xffffu) > (acc.incoming_max >> 16) ? (acc.incoming_max & 0xffffu) : (acc.incoming_max >> 16);
    // wave reduction in a fixed order (xor butterfly): the same inputs always give the same bits
    double dsum = (double)acc.sum;
    uint32_t imax = acc.incoming_max;
#pragma unroll
    for (int w = 32; w >= 1; w >>= 1) {
        dsum += __shfl_xor(dsum, w, 64);
        const uint32_t i2 = (uint32_t)__shfl_xor((int)imax, w, 64);
        imax = i2 > imax ? i2 : imax;
    }
    // what the largest magnitude becomes when it is unscaled and stored (see GradAcc)
    uint32_t smax = imax;
    if (any && inv_scale != 1.0f) {
        if (sizeof(T) == 2) {
            const _Float16 top = __builtin_bit_cast(_Float16, (uint16_t)imax);
            const _Float16 r = half_scale ? top * (_Float16)inv_scale : (_Float16)as_float32((float)top * inv_scale);
            smax = __builtin_bit_cast(uint16_t, r) & 0x7fffu;
        } else {
            smax = __builtin_bit_cast(uint32_t, __builtin_bit_cast(float, imax) * inv_scale) & 0x7fffffffu;
        }
    }
    if (WAVES > 1) {  // the workgroup's waves, added in wave order by one thread
        __shared__ double s_sum[WAVES];
        __shared__ uint32_t s_stored[WAVES], s_incoming[WAVES];
        if (lane == 0) {
            s_sum[wave] = dsum;
            s_stored[wave] = smax;
            s_incoming[wave] = imax;
        }
        __syncthreads();
        if (threadIdx.x == 0) {
#pragma unroll
            for (int w = 1; w < WAVES; ++w) {
                dsum += s_sum[w];
                smax = s_stored[w] > smax ? s_stored[w] : smax;
                imax = s_incoming[w] > imax ? s_incoming[w] : imax;
            }
        }
    }
    if (threadIdx.x == 0) {
        GradPartial part;
        part.sum_squares = dsum;
        part.stored_max = smax;
        part.incoming_max = imax;
        // one ordinary (cached) 16-byte store
        *((gptr<grad_words_t>)reinterpret_cast<grad_words_t*>(partials) + ((blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3))) =
            __builtin_bit_cast(grad_words_t, part);
    }
}

// Fixed-order reduction of `n` partials into `out[blockIdx.x]`: block b takes the b-th contiguous
// slice, thread t every 256th entry of it, then a shared-memory tree.  `per_xcd` != 0: `in` holds the
// partials of `n_groups` workgroups in the slots fsadam_grad_tiles chose (8 rows of per_xcd slots, n = 8 * per_xcd);
// the slots at the end of a row that belong to no workgroup are skipped.  The last step (one block,
// `publish` set) hands the result to the caller's three outputs instead.
__global__ __launch_bounds__(256) void fsadam_grad_reduce(const GradPartial* __restrict__ in, uint32_t n, uint32_t per_block,
                                                          GradPartial* __restrict__ out, int publish, int is_half,
                                                          float* found_inf, double* sum_squares, float* abs_max,
                                                          uint32_t per_xcd, uint32_t n_groups, uint32_t* owner, uint32_t ticket) {
    __shared__ double s_sum[256];
    __shared__ uint32_t s_stored[256];
    __shared__ uint32_t s_incoming[256];
    const uint32_t lo = blockIdx.x * per_block;
    const uint32_t hi = lo + per_block < n ? lo + per_block : n;
    double sum = 0.0;
    uint32_t stored = 0, incoming = 0;
    for (uint32_t i = lo + threadIdx.x; i < hi; i += 256) {
        if (per_xcd) {  // slot i = row * per_xcd + column belongs to workgroup column * 8 + row
            const uint32_t row = i / per_xcd, column = i - row * per_xcd;
            if (column * 8u + row >= n_groups) continue;
        }
        const GradPartial p = in[i];
        sum += p.sum_squares;
        stored = p.stored_max > stored ? p.stored_max : stored;
        incoming = p.incoming_max > incoming ? p.incoming_max : incoming;
    }
    s_sum[threadIdx.x] = sum; s_stored[threadIdx.x] = stored; s_incoming[threadIdx.x] = incoming;
    __syncthreads();
    for (int w = 128; w >= 1; w >>= 1) {
        if ((int)threadIdx.x < w) {
            s_sum[threadIdx.x] += s_sum[threadIdx.x + w];
            s_stored[threadIdx.x] = s_stored[threadIdx.x + w] > s_stored[threadIdx.x] ? s_stored[threadIdx.x + w] : s_stored[threadIdx.x];
            s_incoming[threadIdx.x] = s_incoming[threadIdx.x + w] > s_incoming[threadIdx.x] ? s_incoming[threadIdx.x + w] : s_incoming[threadIdx.x];
        }
        __syncthreads();
    }
    if (threadIdx.x != 0) return;
    if (!publish) {
        out[blockIdx.x].sum_squares = s_sum[0];
        out[blockIdx.x].stored_max = s_stored[0];
        out[blockIdx.x].incoming_max = s_incoming[0];
        return;
    }
    if (owner) {
        // The pass ran on memory that every call on this GPU shares (see fsadam_put_descs).  It is good only if this
        // call still owns that memory and found it free when it began; otherwise another call's kernels ran in between
        // and everything this pass computed is suspect: all three outputs become NaN (a flag that is not zero reads as
        // an overflow to every caller, so the step is skipped rather than taken on a wrong norm).
        const uint32_t holder = __hip_atomic_load(owner, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const bool spoiled = holder != ticket || owner[1] != 0u;
        if (holder == ticket) {  // ours to give back
            owner[1] = 0u;
            __hip_atomic_store(owner, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        if (spoiled) {
            if (found_inf) *found_inf = __builtin_nanf("");
            if (sum_squares) *sum_squares = __builtin_nan("");
            if (abs_max) *abs_max = __builtin_nanf("");
            return;
        }
    }
    const uint32_t inf_pattern = is_half ? 0x7c00u : 0x7f800000u;
    if (s_incoming[0] >= inf_pattern && found_inf) *found_inf = 1.0f;  // set, never cleared: the caller zero-fills it
    if (sum_squares) *sum_squares = s_sum[0];
    // The stored maximum was formed from the largest incoming magnitude, which is right whenever g -> dtype(g * inv_scale)
    // is monotone in |g|.  An infinite or NaN inv_scale breaks that: a zero gradient then stores NaN (0 * inf) while the
    // largest one stores inf.  Squares are never negative, so the sum is NaN exactly when some stored value is NaN:
    // that is when the maximum is NaN too (torch's abs().max() propagates it).
    float top = is_half ? (float)__builtin_bit_cast(_Float16, (uint16_t)s_stored[0]) : __builtin_bit_cast(float, s_stored[0]);
    if (s_sum[0] != s_sum[0]) top = __builtin_nanf("");
    if (abs_max) *abs_max = top;
}

// Rows of a descriptor table handed over in the kernel arguments and written to table[first .. first + count):
// how a table reaches the device without a copy (3 KiB of arguments per launch).
constexpr int kDescsPerPut = 48;
struct DescBatch {
    ChunkDesc rows[kDescsPerPut];
};
// With `owner` set, the first launch of a call (first == 0) also takes possession of the memory the table and the partial results live in:
// owner[0] holds the ticket of the call that is using it (0: free), owner[1] whether that call found it taken when it
// began.  Calls that overlap on one GPU (two streams without an order between them, a replaying graph beside an eager
// call) overwrite each other's table and partials; with the two words each of them finds out at its end (see
// fsadam_grad_reduce) and reports NaN instead of a number that may be wrong.
__global__ __launch_bounds__(64) void fsadam_put_descs(ChunkDesc* __restrict__ table, DescBatch batch, uint32_t first, uint32_t count,
                                                        uint32_t* owner, uint32_t ticket) {
    if (owner && first == 0 && threadIdx.x == 0) {
        const uint32_t before = __hip_atomic_exchange(owner, ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        owner[1] = before != 0u ? 1u : 0u;
    }
    constexpr uint32_t kWords = sizeof(ChunkDesc) / sizeof(uint32_t);
    gptr<uint32_t> out = (gptr<uint32_t>)reinterpret_cast<uint32_t*>(table + first);
    const uint32_t* in = reinterpret_cast<const uint32_t*>(batch.rows);
    for (uint32_t w = threadIdx.x; w < count * kWords; w += 64) out[w] = in[w];
}

}  // namespace
