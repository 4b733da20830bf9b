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
constexpr int64_t kMaxLargeChunk = 1 << 24;   // upper bound (keeps the per-chunk count in 32 bits with room)
constexpr int kBlock = 64;                    // threads per workgroup of the step: one wave64 (128 and 256 measured no faster)

struct alignas(64) ChunkDesc {  // one per chunk; every pointer already points at the chunk's first element
    void* p;
    void* m;
    void* v;
    const void* g;
    void* p_copy;
    uint32_t n;          // elements in this chunk (<= chunk size of its launch)
    uint32_t pad32;
    uint64_t pad;
};
static_assert(sizeof(ChunkDesc) == 64, "descriptor must stay 64 bytes");

// Where the tiles of a launch find their descriptors.  Three classes of descriptors, stored one behind
// the other: large tensors share one among 2^log2_large tiles, middle-sized ones among 2^log2_mid
// tiles, and every tile behind those has a descriptor of its own (small tensors, heads).  A shared
// descriptor keeps the table short (it is sent again whenever a pointer of the list moves) and lets
// neighbouring workgroups fetch the same 64 bytes; its last tiles may lie past the end of the tensor
// and return at once.
struct TileMap {
    uint32_t log2_large, n_large_blocks, n_large_descs;
    uint32_t log2_mid, n_mid_blocks, n_mid_descs;
};
// descriptor index and first element (within the descriptor's chunk) of tile `block`; all operands are
// uniform, so this is scalar arithmetic
__device__ __forceinline__ void locate_tile(const TileMap& map, uint32_t block, uint32_t tile_elems, uint32_t& chunk, uint32_t& off) {
    if (block < map.n_large_blocks) {
        chunk = block >> map.log2_large;
        off = (block & ((1u << map.log2_large) - 1u)) * tile_elems;
    } else if (block - map.n_large_blocks < map.n_mid_blocks) {
        const uint32_t b = block - map.n_large_blocks;
        chunk = map.n_large_descs + (b >> map.log2_mid);
        off = (b & ((1u << map.log2_mid) - 1u)) * tile_elems;
    } else {
        chunk = map.n_large_descs + map.n_mid_descs + (block - map.n_large_blocks - map.n_mid_blocks);
        off = 0u;
    }
}

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

#ifdef __HIPCC__
// One 8- or 16-byte store that leaves for memory as it is issued: device scope (sc1: the L2 writes it through
// instead of keeping a dirty line to evict later) and non-temporal.  The compiler's non-temporal store sets nt
// alone; with sc1 as well a kernel that reads and writes streams moves 2 points more of the HBM rate (measured
// on this part with every combination of the three policy bits, on the loads and on the stores).  Nothing reads
// these bytes again before the kernel ends, so the scope costs nothing.  The address may be any (unaligned-access
// mode), the value any type of 8 or 16 bytes.
// The instruction comes from inline assembly (no builtin sets this combination of bits), so the compiler does not
// see a store: it neither counts it (harmless: waiting for a count that leaves the older loads out still waits for
// them) nor keeps its hands off the data registers for the two wait states this target needs between a store of
// more than 64 bits and a vector instruction that overwrites its data -- the s_nop does.
template <typename V>
__device__ __forceinline__ void store_through(gptr<void> ptr, V value) {
    static_assert(sizeof(V) == 8 || sizeof(V) == 16, "one dwordx2 or dwordx4");
    if constexpr (sizeof(V) == 16) {
        typedef uint32_t words_t __attribute__((ext_vector_type(4)));
        asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(ptr), "v"(__builtin_bit_cast(words_t, value)) : "memory");
    } else {
        typedef uint32_t words_t __attribute__((ext_vector_type(2)));
        asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"(ptr), "v"(__builtin_bit_cast(words_t, value)) : "memory");
    }
}
#endif

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
