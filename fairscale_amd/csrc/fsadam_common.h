// Definitions shared by the kernels and the host code of libfsadam: the chunk descriptor of the
// device-resident table, the per-step scalars, the traits of the dtype combinations.
// Included by fsadam.hip only (one translation unit).
#pragma once

#include <cstdint>

#include "fsadam.h"

namespace {

// --------------------------------------------------------------------------------------------
// shared host/device definitions
// --------------------------------------------------------------------------------------------

constexpr int64_t kLargeThreshold = 131072;   // tensors with at least this many elements share descriptors
constexpr int64_t kMinLargeChunk = 65536;     // elements per shared descriptor, lower bound
constexpr int64_t kMaxLargeChunk = 1 << 24;   // upper bound (keeps the per-chunk count in 32 bits with room); option max_large_chunk lowers it

struct alignas(64) ChunkDesc {  // one per chunk; every pointer already points at the chunk's first element
    void* p;
    void* m;
    void* v;
    const void* g;
    void* p_copy;
    uint32_t n;          // elements in this chunk (<= chunk size of its launch)
    uint32_t vector_ok;  // full tiles of this chunk take the vector path
    uint64_t pad;
};
static_assert(sizeof(ChunkDesc) == 64, "descriptor must stay 64 bytes");

struct StepScalars {
    const float* grad_scale_dev;  // when not NULL the kernel reads the gradient scale here instead of grad_scale
    float b1, b2, one_minus_b1, one_minus_b2;
    float eps, decay, step_size;
    float grad_scale, inv_grad_scale;
    float optim_scale, inv_optim_scale;
    int eps_mode;     // 0: sqrt(v+eps), 1: sqrt(v)+eps
    int fast_scales;  // every scale the mode divides by is a power of two with an exact reciprocal
};

// Pointers read out of the descriptor table would otherwise be generic (flat_* instructions, which
// also tie up the LDS counter); these live in global memory, so say so.
#define FS_GLOBAL __attribute__((address_space(1)))
template <typename T>
using gptr = FS_GLOBAL T*;

template <int MODE>
struct ModeTraits;
template <>
struct ModeTraits<FSADAM_FULL_PRECISION> {
    using P = float; using G = float; using S = float;
    static constexpr bool kCopy = false, kScaled = false;
    static constexpr int kElems = 4;  // elements per lane per group: 16 bytes of the widest stream
};
template <>
struct ModeTraits<FSADAM_MIXED_PRECISION> {
    using P = float; using G = _Float16; using S = float;
    static constexpr bool kCopy = true, kScaled = false;
    static constexpr int kElems = 4;
};
template <>
struct ModeTraits<FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION> {
    using P = _Float16; using G = _Float16; using S = float;
    static constexpr bool kCopy = false, kScaled = false;
    static constexpr int kElems = 4;
};
template <>
struct ModeTraits<FSADAM_PURE_FP16> {
    using P = _Float16; using G = _Float16; using S = _Float16;
    static constexpr bool kCopy = false, kScaled = true;
    static constexpr int kElems = 8;
};

template <>
struct ModeTraits<FSADAM_FULL_PRECISION_FP16_COPY> {
    using P = float; using G = float; using S = float;
    static constexpr bool kCopy = true, kScaled = false;
    static constexpr int kElems = 4;
};

constexpr int mode_elems(int mode) { return mode == FSADAM_PURE_FP16 ? 8 : 4; }
constexpr bool mode_has_copy(int mode) { return mode == FSADAM_MIXED_PRECISION || mode == FSADAM_FULL_PRECISION_FP16_COPY; }

}  // namespace
