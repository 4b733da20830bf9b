// Microbenchmarks of the memory-access structures the Adam kernels were chosen among (MI355X, gfx950).
// Not part of the product: built into libfsadam_membench.so, driven by `bench.py --micro`, which times
// the launches with HIP events and prints a table.  Every kernel moves the streams of an Adam step with
// trivial arithmetic (two multiply-adds per element), so that what is measured is the memory system:
//   * four fp32 streams p, m, v, g of `n` elements, read (all four) and written back (p, m, v): 28 bytes
//     per element, the FULL_PRECISION shape; or
//   * the MEMORY_EFFICIENT shape: p, g fp16 (2 bytes), m, v fp32: 12 bytes read, 10 written per element.
// One entry point launches one variant once on the caller's stream; nothing is allocated here.
#include <hip/hip_runtime.h>

#include <cstdint>

#define FS_GLOBAL __attribute__((address_space(1)))
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));

namespace {

template <bool NT, typename T>
__device__ __forceinline__ T ld(FS_GLOBAL const T* p) {
    return NT ? __builtin_nontemporal_load(p) : *p;
}
template <bool NT, typename T>
__device__ __forceinline__ void st(FS_GLOBAL T* p, T v) {
    if (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// What the write-only kernels store: zeros, or (pattern != 0) floats in [1, 2) whose mantissa bits are a hash of the
// position -- the bandwidth of this part depends on the data (see run_micro in bench.py), and optimizer state is not zeros.
__device__ __forceinline__ f4 fill_value(int64_t i, int pattern) {
    if (!pattern) return f4{0.f, 0.f, 0.f, 0.f};
    uint32_t h = (uint32_t)i * 2654435761u + 0x9e3779b9u;
    f4 out;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        out[k] = __builtin_bit_cast(float, (h & 0x007fffffu) | 0x3f800000u);
    }
    return out;
}

// the stand-in for the update: enough arithmetic to keep every loaded value alive, nothing more
__device__ __forceinline__ void fake_update(f4& p, f4& m, f4& v, f4 g) {
    m = m * 0.9f + g * 0.1f;
    v = v * 0.999f + g * g * 0.001f;
    p = p - m * 0.001f;
}

// ---- variant 0/2: one-shot tiles.  One workgroup = one wave64 = 64 quads per stream, then it exits.
template <bool NT>
__global__ __launch_bounds__(64) void mb_oneshot(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + i;
    f4 a = ld<NT>((FS_GLOBAL const f4*)p), b = ld<NT>((FS_GLOBAL const f4*)m), c = ld<NT>((FS_GLOBAL const f4*)v),
       d = ld<NT>((FS_GLOBAL const f4*)g_ + i);
    fake_update(a, b, c, d);
    st<NT>(m, b);
    st<NT>(v, c);
    st<NT>(p, a);
}

// ---- variant 1: persistent workgroups of 256 threads in a grid-stride loop (grid = CUs x workgroups per CU).
__global__ __launch_bounds__(256) void mb_gridstride(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq) {
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_;
    FS_GLOBAL const f4* g = (FS_GLOBAL const f4*)g_;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < nq; i += (int64_t)gridDim.x * 256) {
        f4 a = ld<true>((FS_GLOBAL const f4*)p + i), b = ld<true>((FS_GLOBAL const f4*)m + i), c = ld<true>((FS_GLOBAL const f4*)v + i),
           d = ld<true>(g + i);
        fake_update(a, b, c, d);
        st<true>(m + i, b);
        st<true>(v + i, c);
        st<true>(p + i, a);
    }
}

// ---- variants 3/4: the pointers come from a table of 64-byte descriptors in device memory (one per chunk of
// `tiles_per_desc` tiles), as in the multi-tensor step.
struct alignas(64) MbDesc {
    f4* p;
    f4* m;
    f4* v;
    const f4* g;
    uint64_t nq;  // quads in this chunk
    uint64_t pad[3];
};

// 4: one scalar load of the whole descriptor (uniform address, constant address space) per wave -- the product's way
__global__ __launch_bounds__(64) void mb_table_scalar(const MbDesc* table, uint32_t log2_tiles) {
    const uint32_t chunk = blockIdx.x >> log2_tiles, tile = blockIdx.x & ((1u << log2_tiles) - 1u);
    typedef uint32_t words_t __attribute__((ext_vector_type(16)));
    const words_t raw = *reinterpret_cast<const __attribute__((address_space(4))) words_t*>((const __attribute__((address_space(4))) MbDesc*)table + chunk);
    const MbDesc d = __builtin_bit_cast(MbDesc, raw);
    const uint64_t i = (uint64_t)tile * 64 + threadIdx.x;
    if (i >= d.nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)d.p + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)d.m + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)d.v + i;
    f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
       e = ld<true>((FS_GLOBAL const f4*)d.g + i);
    fake_update(a, b, c, e);
    st<true>(m, b);
    st<true>(v, c);
    st<true>(p, a);
}

// 3: the descriptor is staged in LDS by the workgroup's first lanes, the workgroup synchronises, and every lane reads
// the pointers from LDS -- the structure of a launcher whose metadata lives in shared memory
__global__ __launch_bounds__(64) void mb_table_lds(const MbDesc* table, uint32_t log2_tiles) {
    __shared__ MbDesc staged;
    const uint32_t chunk = blockIdx.x >> log2_tiles, tile = blockIdx.x & ((1u << log2_tiles) - 1u);
    if (threadIdx.x < 16) reinterpret_cast<uint32_t*>(&staged)[threadIdx.x] = reinterpret_cast<const uint32_t*>(table + chunk)[threadIdx.x];
    __syncthreads();
    const uint64_t i = (uint64_t)tile * 64 + threadIdx.x;
    if (i >= staged.nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)staged.p + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)staged.m + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)staged.v + i;
    f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
       e = ld<true>((FS_GLOBAL const f4*)staged.g + i);
    fake_update(a, b, c, e);
    st<true>(m, b);
    st<true>(v, c);
    st<true>(p, a);
}

// ---- variants 30-33: the two ways to the descriptor again, with the stores written through (sc1 nt) as the Adam kernels
// issue them, for the 28-byte shape (30 scalar load, 31 staged in LDS) and the MEMORY_EFFICIENT shape (32, 33; the table
// then holds p and g advanced as fp16 streams, see mb_fill_table).  Defined after st_policy below.
template <bool LDS, bool MEMEFF>
__global__ __launch_bounds__(64) void mb_table_through(const MbDesc* table, uint32_t log2_tiles);

// ---- variants 5/6: the fp32 streams one direction at a time (one-shot tiles).
__global__ __launch_bounds__(64) void mb_read4(const f4* p_, const f4* m_, const f4* v_, const f4* g_, int64_t nq, float* sink) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 s = ld<true>((FS_GLOBAL const f4*)p_ + i) + ld<true>((FS_GLOBAL const f4*)m_ + i) + ld<true>((FS_GLOBAL const f4*)v_ + i) +
                 ld<true>((FS_GLOBAL const f4*)g_ + i);
    if (s[0] + s[1] + s[2] + s[3] == 12345.678f) *sink = 1.0f;  // never true for the zero-filled buffers: keeps the loads
}
__global__ __launch_bounds__(64) void mb_write3(f4* p_, f4* m_, f4* v_, int64_t nq, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 val = fill_value(i, pattern);
    st<true>((FS_GLOBAL f4*)m_ + i, val);
    st<true>((FS_GLOBAL f4*)v_ + i, val);
    st<true>((FS_GLOBAL f4*)p_ + i, val);
}

// ---- variants 7/8/9: the MEMORY_EFFICIENT shape (4 elements per lane: 8 bytes of the fp16 streams, 16 of the fp32 ones):
// reads only (12 B/elt), writes only (10 B/elt), both (22 B/elt).  `n4` = groups of 4 elements.
__global__ __launch_bounds__(64) void mb_memeff_read(const f2* p_, const f4* m_, const f4* v_, const f2* g_, int64_t n4, float* sink) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    const f2 a = ld<true>((FS_GLOBAL const f2*)p_ + i), d = ld<true>((FS_GLOBAL const f2*)g_ + i);
    const f4 s = ld<true>((FS_GLOBAL const f4*)m_ + i) + ld<true>((FS_GLOBAL const f4*)v_ + i);
    if (s[0] + s[1] + s[2] + s[3] + a[0] + a[1] + d[0] + d[1] == 12345.678f) *sink = 1.0f;
}
__global__ __launch_bounds__(64) void mb_memeff_write(f2* p_, f4* m_, f4* v_, int64_t n4, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    const f4 val = fill_value(i, pattern);
    const f2 half = {val[0], val[1]};
    st<true>((FS_GLOBAL f4*)m_ + i, val);
    st<true>((FS_GLOBAL f4*)v_ + i, val);
    st<true>((FS_GLOBAL f2*)p_ + i, half);
}
__global__ __launch_bounds__(64) void mb_memeff_both(f2* p_, f4* m_, f4* v_, const f2* g_, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    f2 a = ld<true>((FS_GLOBAL const f2*)p_ + i);
    const f2 d = ld<true>((FS_GLOBAL const f2*)g_ + i);
    f4 b = ld<true>((FS_GLOBAL const f4*)m_ + i), c = ld<true>((FS_GLOBAL const f4*)v_ + i);
    const f4 g = {d[0], d[1], d[0], d[1]};
    b = b * 0.9f + g * 0.1f;
    c = c * 0.999f + g * g * 0.001f;
    a[0] -= b[0] * 0.001f;
    a[1] -= b[1] * 0.001f;
    st<true>((FS_GLOBAL f4*)m_ + i, b);
    st<true>((FS_GLOBAL f4*)v_ + i, c);
    st<true>((FS_GLOBAL f2*)p_ + i, a);
}

// ---- variants 10-13: what else could be done about the write side.
// 10: ONE stream written (a fill); 11: three streams with plain (temporal) stores; 12: three streams, every wave
// writes four consecutive vectors per stream (4 KiB bursts); 13: the 28-byte shape with four vectors per lane and
// stream: all sixteen loads first, then all twelve stores (longer same-direction bursts per wave).
__global__ __launch_bounds__(64) void mb_write1(f4* p_, int64_t nq, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 val = fill_value(i, pattern);
    st<true>((FS_GLOBAL f4*)p_ + i, val);
}
__global__ __launch_bounds__(64) void mb_write3_temporal(f4* p_, f4* m_, f4* v_, int64_t nq, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 val = fill_value(i, pattern);
    st<false>((FS_GLOBAL f4*)m_ + i, val);
    st<false>((FS_GLOBAL f4*)v_ + i, val);
    st<false>((FS_GLOBAL f4*)p_ + i, val);
}
__global__ __launch_bounds__(64) void mb_write3_bursts(f4* p_, f4* m_, f4* v_, int64_t nq, int pattern) {
    const int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const f4 val = fill_value(base, pattern);
#pragma unroll
    for (int k = 0; k < 4; ++k) if (base + k * 64 < nq) st<true>((FS_GLOBAL f4*)m_ + base + k * 64, val);
#pragma unroll
    for (int k = 0; k < 4; ++k) if (base + k * 64 < nq) st<true>((FS_GLOBAL f4*)v_ + base + k * 64, val);
#pragma unroll
    for (int k = 0; k < 4; ++k) if (base + k * 64 < nq) st<true>((FS_GLOBAL f4*)p_ + base + k * 64, val);
}
__global__ __launch_bounds__(64) void mb_oneshot_x4(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq) {
    const int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (base + 192 >= nq) return;  // the ragged end is left out: a handful of quads in 4e8
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + base;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + base;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + base;
    FS_GLOBAL const f4* g = (FS_GLOBAL const f4*)g_ + base;
    f4 a[4], b[4], c[4], d[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        a[k] = ld<true>((FS_GLOBAL const f4*)p + k * 64); b[k] = ld<true>((FS_GLOBAL const f4*)m + k * 64);
        c[k] = ld<true>((FS_GLOBAL const f4*)v + k * 64); d[k] = ld<true>(g + k * 64);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) fake_update(a[k], b[k], c[k], d[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(m + k * 64, b[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(v + k * 64, c[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(p + k * 64, a[k]);
}

// ---- variants 14/15: one-shot tiles in an XCD-aware order.  Workgroup b runs on XCD b % 8 (hardware dispatch is
// round-robin over the eight XCDs); within every group of 8 * R workgroups, workgroup b takes tile
// (b % 8) * R + (b / 8) % R, so that each XCD (each L2) works through runs of R consecutive tiles.
__device__ __forceinline__ int64_t xcd_tile(int64_t b, int log2_run) {
    const int64_t span = (int64_t)8 << log2_run, group = b / span, in = b % span;
    return group * span + ((in & 7) << log2_run) + (in >> 3);
}
__global__ __launch_bounds__(64) void mb_oneshot_xcd(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq, int log2_run) {
    const int64_t i = xcd_tile(blockIdx.x, log2_run) * 64 + threadIdx.x;
    if (i >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + i;
    f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
       d = ld<true>((FS_GLOBAL const f4*)g_ + i);
    fake_update(a, b, c, d);
    st<true>(m, b);
    st<true>(v, c);
    st<true>(p, a);
}
__global__ __launch_bounds__(64) void mb_memeff_both_xcd(f2* p_, f4* m_, f4* v_, const f2* g_, int64_t n4, int log2_run) {
    const int64_t i = xcd_tile(blockIdx.x, log2_run) * 64 + threadIdx.x;
    if (i >= n4) return;
    f2 a = ld<true>((FS_GLOBAL const f2*)p_ + i);
    const f2 d = ld<true>((FS_GLOBAL const f2*)g_ + i);
    f4 b = ld<true>((FS_GLOBAL const f4*)m_ + i), c = ld<true>((FS_GLOBAL const f4*)v_ + i);
    const f4 g = {d[0], d[1], d[0], d[1]};
    b = b * 0.9f + g * 0.1f;
    c = c * 0.999f + g * g * 0.001f;
    a[0] -= b[0] * 0.001f;
    a[1] -= b[1] * 0.001f;
    st<true>((FS_GLOBAL f4*)m_ + i, b);
    st<true>((FS_GLOBAL f4*)v_ + i, c);
    st<true>((FS_GLOBAL f2*)p_ + i, a);
}
__global__ __launch_bounds__(64) void mb_write3_xcd(f4* p_, f4* m_, f4* v_, int64_t nq, int log2_run, int pattern) {
    const int64_t i = xcd_tile(blockIdx.x, log2_run) * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 val = fill_value(i, pattern);
    st<true>((FS_GLOBAL f4*)m_ + i, val);
    st<true>((FS_GLOBAL f4*)v_ + i, val);
    st<true>((FS_GLOBAL f4*)p_ + i, val);
}

// ---- variants 17/18/19: device-wide read and write phases set by the clock.  Every wave reads the constant-rate real-time
// counter (the same for all waves of the device), issues its loads only in the first `split` ticks of every `period` ticks and
// its stores only in the rest, so that at any instant the whole device moves data in one direction.  Waits are bounded.
__device__ __forceinline__ void wait_phase(uint32_t period, uint32_t split, bool writing) {
    for (int spin = 0; spin < 100000; ++spin) {
        const uint32_t t = (uint32_t)(wall_clock64() % period);
        if ((t >= split) == writing) return;
        __builtin_amdgcn_s_sleep(1);
    }
}
__global__ __launch_bounds__(64) void mb_oneshot_phased(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq, uint32_t period, uint32_t split) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + i;
    wait_phase(period, split, false);
    f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
       d = ld<true>((FS_GLOBAL const f4*)g_ + i);
    fake_update(a, b, c, d);
    // the wait must not be hoisted above the loads' return: it depends on a loaded value
    if (a[0] == 12345.678f) return;
    wait_phase(period, split, true);
    st<true>(m, b);
    st<true>(v, c);
    st<true>(p, a);
}
__global__ __launch_bounds__(64) void mb_oneshot_x4_phased(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq, uint32_t period, uint32_t split) {
    const int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (base + 192 >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + base;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + base;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + base;
    FS_GLOBAL const f4* g = (FS_GLOBAL const f4*)g_ + base;
    f4 a[4], b[4], c[4], d[4];
    wait_phase(period, split, false);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        a[k] = ld<true>((FS_GLOBAL const f4*)p + k * 64); b[k] = ld<true>((FS_GLOBAL const f4*)m + k * 64);
        c[k] = ld<true>((FS_GLOBAL const f4*)v + k * 64); d[k] = ld<true>(g + k * 64);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) fake_update(a[k], b[k], c[k], d[k]);
    if (a[0][0] + a[1][0] + a[2][0] + a[3][0] == 12345.678f) return;
    wait_phase(period, split, true);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(m + k * 64, b[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(v + k * 64, c[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st<true>(p + k * 64, a[k]);
}
__global__ __launch_bounds__(64) void mb_memeff_both_phased(f2* p_, f4* m_, f4* v_, const f2* g_, int64_t n4, uint32_t period, uint32_t split) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    wait_phase(period, split, false);
    f2 a = ld<true>((FS_GLOBAL const f2*)p_ + i);
    const f2 d = ld<true>((FS_GLOBAL const f2*)g_ + i);
    f4 b = ld<true>((FS_GLOBAL const f4*)m_ + i), c = ld<true>((FS_GLOBAL const f4*)v_ + i);
    const f4 g = {d[0], d[1], d[0], d[1]};
    b = b * 0.9f + g * 0.1f;
    c = c * 0.999f + g * g * 0.001f;
    a[0] -= b[0] * 0.001f;
    a[1] -= b[1] * 0.001f;
    if (a[0] == 12345.678f) return;
    wait_phase(period, split, true);
    st<true>((FS_GLOBAL f4*)m_ + i, b);
    st<true>((FS_GLOBAL f4*)v_ + i, c);
    st<true>((FS_GLOBAL f2*)p_ + i, a);
}

// ---- variants 20/21: the cache-policy bits of the memory instructions.  gfx950 loads and stores carry three bits: sc0 and
// sc1 (the scope the access must be coherent at: wave, workgroup, device, system) and nt (non-temporal); the compiler's
// non-temporal builtins set nt alone.  The MEMORY_EFFICIENT shape with the stores (20) or the loads (21) issued from inline
// assembly with every combination of the three: POLICY bit 0 = sc0, bit 1 = sc1, bit 2 = nt.
#define MB_POLICY_CASES(X) X(0, "") X(1, " sc0") X(2, " sc1") X(3, " sc0 sc1") X(4, " nt") X(5, " sc0 nt") X(6, " sc1 nt") X(7, " sc0 sc1 nt")
template <int POLICY>
__device__ __forceinline__ void st_policy(FS_GLOBAL f4* p, f4 v) {
#define X(N, BITS) if constexpr (POLICY == N) asm volatile("global_store_dwordx4 %0, %1, off" BITS "\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
    MB_POLICY_CASES(X)
#undef X
}
template <int POLICY>
__device__ __forceinline__ void st_policy(FS_GLOBAL f2* p, f2 v) {
#define X(N, BITS) if constexpr (POLICY == N) asm volatile("global_store_dwordx2 %0, %1, off" BITS ::"v"(p), "v"(v) : "memory");
    MB_POLICY_CASES(X)
#undef X
}
// The four loads of a MEMORY_EFFICIENT tile and the wait for them in ONE statement: the compiler neither counts loads it
// did not issue nor knows when their results arrive, so nothing may sit between them and their wait (outputs are
// early-clobber: no result register doubles as an address).
template <int POLICY>
__device__ __forceinline__ void ld4_policy(f2& a, f2& d, f4& b, f4& c, FS_GLOBAL const f2* pa, FS_GLOBAL const f2* pd, FS_GLOBAL const f4* pb,
                                           FS_GLOBAL const f4* pc) {
#define X(N, BITS)                                                                                                                        \
    if constexpr (POLICY == N)                                                                                                            \
        asm volatile("global_load_dwordx2 %0, %4, off" BITS "\n\tglobal_load_dwordx2 %1, %5, off" BITS "\n\tglobal_load_dwordx4 %2, %6, off" BITS \
                     "\n\tglobal_load_dwordx4 %3, %7, off" BITS "\n\ts_waitcnt vmcnt(0)"                                               \
                     : "=&v"(a), "=&v"(d), "=&v"(b), "=&v"(c)                                                                              \
                     : "v"(pa), "v"(pd), "v"(pb), "v"(pc)                                                                                  \
                     : "memory");
    MB_POLICY_CASES(X)
#undef X
}
template <int LOADS, int STORES>  // a policy, or -1 for the compiler's non-temporal builtin
__global__ __launch_bounds__(64) void mb_memeff_both_policy(f2* p_, f4* m_, f4* v_, const f2* g_, int64_t n4) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    f2 a, d;
    f4 b, c;
    if constexpr (LOADS < 0) {
        a = ld<true>((FS_GLOBAL const f2*)p_ + i);
        d = ld<true>((FS_GLOBAL const f2*)g_ + i);
        b = ld<true>((FS_GLOBAL const f4*)m_ + i);
        c = ld<true>((FS_GLOBAL const f4*)v_ + i);
    } else {
        ld4_policy<LOADS>(a, d, b, c, (FS_GLOBAL const f2*)p_ + i, (FS_GLOBAL const f2*)g_ + i, (FS_GLOBAL const f4*)m_ + i, (FS_GLOBAL const f4*)v_ + i);
    }
    const f4 g = {d[0], d[1], d[0], d[1]};
    b = b * 0.9f + g * 0.1f;
    c = c * 0.999f + g * g * 0.001f;
    a[0] -= b[0] * 0.001f;
    a[1] -= b[1] * 0.001f;
    if constexpr (STORES < 0) {
        st<true>((FS_GLOBAL f4*)m_ + i, b);
        st<true>((FS_GLOBAL f4*)v_ + i, c);
        st<true>((FS_GLOBAL f2*)p_ + i, a);
    } else {
        st_policy<STORES>((FS_GLOBAL f4*)m_ + i, b);
        st_policy<STORES>((FS_GLOBAL f4*)v_ + i, c);
        st_policy<STORES>((FS_GLOBAL f2*)p_ + i, a);
    }
}

template <bool LDS, bool MEMEFF>
__global__ __launch_bounds__(64) void mb_table_through(const MbDesc* table, uint32_t log2_tiles) {
    const uint32_t chunk = blockIdx.x >> log2_tiles, tile = blockIdx.x & ((1u << log2_tiles) - 1u);
    MbDesc d;
    if constexpr (LDS) {
        __shared__ MbDesc staged;
        if (threadIdx.x < 16) reinterpret_cast<uint32_t*>(&staged)[threadIdx.x] = reinterpret_cast<const uint32_t*>(table + chunk)[threadIdx.x];
        __syncthreads();
        d = staged;
    } else {
        typedef uint32_t words_t __attribute__((ext_vector_type(16)));
        const words_t raw = *reinterpret_cast<const __attribute__((address_space(4))) words_t*>((const __attribute__((address_space(4))) MbDesc*)table + chunk);
        d = __builtin_bit_cast(MbDesc, raw);
    }
    const uint64_t i = (uint64_t)tile * 64 + threadIdx.x;
    if (i >= d.nq) return;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)d.m + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)d.v + i;
    if constexpr (MEMEFF) {
        FS_GLOBAL f2* p = (FS_GLOBAL f2*)reinterpret_cast<f2*>(d.p) + i;
        f2 a = ld<true>((FS_GLOBAL const f2*)p);
        const f2 e = ld<true>((FS_GLOBAL const f2*)reinterpret_cast<const f2*>(d.g) + i);
        f4 b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v);
        const f4 g = {e[0], e[1], e[0], e[1]};
        b = b * 0.9f + g * 0.1f;
        c = c * 0.999f + g * g * 0.001f;
        a[0] -= b[0] * 0.001f;
        a[1] -= b[1] * 0.001f;
        st_policy<6>(m, b);
        st_policy<6>(v, c);
        st_policy<6>(p, a);
    } else {
        FS_GLOBAL f4* p = (FS_GLOBAL f4*)d.p + i;
        f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
           e = ld<true>((FS_GLOBAL const f4*)d.g + i);
        fake_update(a, b, c, e);
        st_policy<6>(m, b);
        st_policy<6>(v, c);
        st_policy<6>(p, a);
    }
}

// 28: two streams of 16 bytes per lane written, 23: the write side of the MEMORY_EFFICIENT shape alone, 24: the 28-byte shape, 25: the 28-byte shape with four vectors per
// lane (all loads, then all stores) -- each with the stores under policy STORES and the loads from the builtin.
template <int STORES>
__global__ __launch_bounds__(64) void mb_memeff_write_policy(f2* p_, f4* m_, f4* v_, int64_t n4, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n4) return;
    const f4 val = fill_value(i, pattern);
    const f2 half = {val[0], val[1]};
    st_policy<STORES>((FS_GLOBAL f4*)m_ + i, val);
    st_policy<STORES>((FS_GLOBAL f4*)v_ + i, val);
    st_policy<STORES>((FS_GLOBAL f2*)p_ + i, half);
}
template <int STORES>  // two streams of 16 bytes per lane: what zeroing fp16 or fp32 state writes
__global__ __launch_bounds__(64) void mb_write2_policy(f4* m_, f4* v_, int64_t nq, int pattern) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    const f4 val = fill_value(i, pattern);
    st_policy<STORES>((FS_GLOBAL f4*)m_ + i, val);
    st_policy<STORES>((FS_GLOBAL f4*)v_ + i, val);
}
template <int STORES>
__global__ __launch_bounds__(64) void mb_oneshot_policy(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + i;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + i;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + i;
    f4 a = ld<true>((FS_GLOBAL const f4*)p), b = ld<true>((FS_GLOBAL const f4*)m), c = ld<true>((FS_GLOBAL const f4*)v),
       d = ld<true>((FS_GLOBAL const f4*)g_ + i);
    fake_update(a, b, c, d);
    st_policy<STORES>(m, b);
    st_policy<STORES>(v, c);
    st_policy<STORES>(p, a);
}
template <int STORES>
__global__ __launch_bounds__(64) void mb_oneshot_x4_policy(f4* p_, f4* m_, f4* v_, const f4* g_, int64_t nq) {
    const int64_t base = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (base + 192 >= nq) return;
    FS_GLOBAL f4* p = (FS_GLOBAL f4*)p_ + base;
    FS_GLOBAL f4* m = (FS_GLOBAL f4*)m_ + base;
    FS_GLOBAL f4* v = (FS_GLOBAL f4*)v_ + base;
    FS_GLOBAL const f4* g = (FS_GLOBAL const f4*)g_ + base;
    f4 a[4], b[4], c[4], d[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        a[k] = ld<true>((FS_GLOBAL const f4*)p + k * 64); b[k] = ld<true>((FS_GLOBAL const f4*)m + k * 64);
        c[k] = ld<true>((FS_GLOBAL const f4*)v + k * 64); d[k] = ld<true>(g + k * 64);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) fake_update(a[k], b[k], c[k], d[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st_policy<STORES>(m + k * 64, b[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st_policy<STORES>(v + k * 64, c[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) st_policy<STORES>(p + k * 64, a[k]);
}

// 26: the MEMORY_EFFICIENT shape with everything that can be varied around write-through stores: policy of the stores,
// TILES consecutive tiles per wave (all loads, then all stores), BLOCK threads per workgroup (64, or 256 = four waves that
// cover 4 KiB per fp32 stream between them), tiles in runs of 2^log2_run per XCD (0: dispatch order).
template <int STORES, int TILES, int BLOCK>
__global__ __launch_bounds__(BLOCK) void mb_memeff_lab(f2* p_, f4* m_, f4* v_, const f2* g_, int64_t n4, int log2_run) {
    const int64_t tile = log2_run ? xcd_tile(blockIdx.x, log2_run) : (int64_t)blockIdx.x;
    const int64_t base = tile * (BLOCK * TILES) + threadIdx.x;
    if (base + (TILES - 1) * BLOCK >= n4) return;  // the ragged end is left out
    f2 a[TILES], d[TILES];
    f4 b[TILES], c[TILES];
#pragma unroll
    for (int k = 0; k < TILES; ++k) {
        a[k] = ld<true>((FS_GLOBAL const f2*)p_ + base + k * BLOCK);
        d[k] = ld<true>((FS_GLOBAL const f2*)g_ + base + k * BLOCK);
        b[k] = ld<true>((FS_GLOBAL const f4*)m_ + base + k * BLOCK);
        c[k] = ld<true>((FS_GLOBAL const f4*)v_ + base + k * BLOCK);
    }
#pragma unroll
    for (int k = 0; k < TILES; ++k) {
        const f4 g = {d[k][0], d[k][1], d[k][0], d[k][1]};
        b[k] = b[k] * 0.9f + g * 0.1f;
        c[k] = c[k] * 0.999f + g * g * 0.001f;
        a[k][0] -= b[k][0] * 0.001f;
        a[k][1] -= b[k][1] * 0.001f;
    }
#pragma unroll
    for (int k = 0; k < TILES; ++k) st_policy<STORES>((FS_GLOBAL f4*)m_ + base + k * BLOCK, b[k]);
#pragma unroll
    for (int k = 0; k < TILES; ++k) st_policy<STORES>((FS_GLOBAL f4*)v_ + base + k * BLOCK, c[k]);
#pragma unroll
    for (int k = 0; k < TILES; ++k) st_policy<STORES>((FS_GLOBAL f2*)p_ + base + k * BLOCK, a[k]);
}

// 29: the MEMORY_EFFICIENT shape with half the bytes per wave: 8 bytes per lane of the fp32 streams, 4 of the fp16 ones
// (128 elements per wave instead of 256), stores written through.
__global__ __launch_bounds__(64) void mb_memeff_half_tile(float* p_, f2* m_, f2* v_, const float* g_, int64_t n2) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i >= n2) return;
    float a = ld<true>((FS_GLOBAL const float*)p_ + i);          // two halves
    const float d = ld<true>((FS_GLOBAL const float*)g_ + i);    // two halves
    f2 b = ld<true>((FS_GLOBAL const f2*)m_ + i), c = ld<true>((FS_GLOBAL const f2*)v_ + i);
    const f2 g = {d, d};
    b = b * 0.9f + g * 0.1f;
    c = c * 0.999f + g * g * 0.001f;
    a -= b[0] * 0.001f;
    asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"((FS_GLOBAL f2*)m_ + i), "v"(b) : "memory");
    asm volatile("global_store_dwordx2 %0, %1, off sc1 nt" ::"v"((FS_GLOBAL f2*)v_ + i), "v"(c) : "memory");
    asm volatile("global_store_dword %0, %1, off sc1 nt" ::"v"((FS_GLOBAL float*)p_ + i), "v"(a) : "memory");
}

__global__ __launch_bounds__(64) void mb_copy(f4* dst_, const f4* src_, int64_t n_quads) {
    const int64_t i = (int64_t)blockIdx.x * 64 + threadIdx.x;
    if (i < n_quads) __builtin_nontemporal_store(__builtin_nontemporal_load((FS_GLOBAL const f4*)src_ + i), (FS_GLOBAL f4*)dst_ + i);
}

// fills a table of descriptors over four flat buffers, `chunk_q` quads each (runs once, outside the timing)
// half_pg: p and g are fp16 streams (8 bytes per group of four elements), as in the MEMORY_EFFICIENT shape
__global__ void mb_fill_table(MbDesc* table, f4* p, f4* m, f4* v, const f4* g, uint64_t nq, uint64_t chunk_q, uint32_t n_desc, int half_pg) {
    const uint32_t k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_desc) return;
    const uint64_t first = (uint64_t)k * chunk_q;
    MbDesc d = {};
    d.m = m + first; d.v = v + first;
    if (half_pg) { d.p = reinterpret_cast<f4*>(reinterpret_cast<f2*>(p) + first); d.g = reinterpret_cast<const f4*>(reinterpret_cast<const f2*>(g) + first); }
    else { d.p = p + first; d.g = g + first; }
    d.nq = nq - first < chunk_q ? nq - first : chunk_q;
    table[k] = d;
}

}  // namespace

namespace {
int g_pattern = 0;
}

extern "C" {

// What the write-only variants store from now on: 0 zeros (default), 1 floats with hashed mantissas.
void fsadam_membench_set_pattern(int pattern) { g_pattern = pattern != 0; }

// Bytes the caller must provide for the descriptor table of variants 3 and 4 (chunks of 2^16 quads).
int64_t fsadam_membench_table_bytes(int64_t numel) {
    const int64_t nq = numel / 4, chunk_q = 1 << 16;
    return ((nq + chunk_q - 1) / chunk_q) * (int64_t)sizeof(MbDesc);
}

// Launches variant `kind` once over `numel` elements (a multiple of 4) on `stream`.  p, m, v, g: device buffers of
// numel floats (the MEMORY_EFFICIENT variants use the first half of p and g as fp16).  lds_bytes: untouched LDS given to
// every workgroup (caps residency).  param: variant 1: workgroups per compute unit; variants 14-16: log2 of the run length in tiles; variants 17-19: the period in 10 ns ticks.  table: device memory of
// fsadam_membench_table_bytes(numel) bytes for variants 3, 4, 30-33, -1 and -2 (-1 fills it for the fp32 shape, -2 for the
// MEMORY_EFFICIENT shape of variants 32 and 33; do that before them).
// Returns 0, or -1 for an unknown kind / bad argument, -2 for a launch error.
int fsadam_membench_launch(int kind, void* p, void* m, void* v, void* g, int64_t numel, int lds_bytes, int param, void* table, void* sink,
                           void* stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (numel <= 0 || (numel & 3) || !p || !m || !v || !g) return -1;
    const int64_t nq = numel / 4;
    const int64_t grid64 = (nq + 63) / 64;
    if (grid64 > 0x7ffffff0) return -1;
    f4 *P = (f4*)p, *M = (f4*)m, *V = (f4*)v;
    const f4* G = (const f4*)g;
    const size_t lds = (size_t)lds_bytes;
    const int64_t chunk_q = 1 << 16;
    const uint32_t n_desc = (uint32_t)((nq + chunk_q - 1) / chunk_q);
    switch (kind) {
        case -1:
        case -2:
            if (!table) return -1;
            hipLaunchKernelGGL(mb_fill_table, dim3((n_desc + 255) / 256), dim3(256), 0, stream, (MbDesc*)table, P, M, V, G, (uint64_t)nq, (uint64_t)chunk_q, n_desc,
                               kind == -2 ? 1 : 0);
            break;
        case 30:
        case 31:
        case 32:
        case 33: {
            if (!table) return -1;
            const uint32_t log2_tiles = 10, grid = n_desc << log2_tiles;
            if (kind == 30) hipLaunchKernelGGL((mb_table_through<false, false>), dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            else if (kind == 31) hipLaunchKernelGGL((mb_table_through<true, false>), dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            else if (kind == 32) hipLaunchKernelGGL((mb_table_through<false, true>), dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            else hipLaunchKernelGGL((mb_table_through<true, true>), dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            break;
        }
        case 0: hipLaunchKernelGGL(mb_oneshot<true>, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, G, nq); break;
        case 1: {
            int dev = 0, cus = 256;
            if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return -2;
            hipLaunchKernelGGL(mb_gridstride, dim3((uint32_t)(cus * (param > 0 ? param : 8))), dim3(256), lds, stream, P, M, V, G, nq);
            break;
        }
        case 2: hipLaunchKernelGGL(mb_oneshot<false>, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, G, nq); break;
        case 3:
        case 4: {
            if (!table) return -1;
            const uint32_t log2_tiles = 10;  // 2^16 quads per descriptor / 64 quads per tile
            const uint32_t grid = n_desc << log2_tiles;
            if (kind == 3) hipLaunchKernelGGL(mb_table_lds, dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            else hipLaunchKernelGGL(mb_table_scalar, dim3(grid), dim3(64), lds, stream, (const MbDesc*)table, log2_tiles);
            break;
        }
        case 5: hipLaunchKernelGGL(mb_read4, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, G, nq, (float*)sink); break;
        case 6: hipLaunchKernelGGL(mb_write3, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, nq, g_pattern); break;
        case 7: hipLaunchKernelGGL(mb_memeff_read, dim3((uint32_t)grid64), dim3(64), lds, stream, (const f2*)p, M, V, (const f2*)g, nq, (float*)sink); break;
        case 8: hipLaunchKernelGGL(mb_memeff_write, dim3((uint32_t)grid64), dim3(64), lds, stream, (f2*)p, M, V, nq, g_pattern); break;
        case 9: hipLaunchKernelGGL(mb_memeff_both, dim3((uint32_t)grid64), dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq); break;
        case 10: hipLaunchKernelGGL(mb_write1, dim3((uint32_t)grid64), dim3(64), lds, stream, P, nq, g_pattern); break;
        case 11: hipLaunchKernelGGL(mb_write3_temporal, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, nq, g_pattern); break;
        case 12: hipLaunchKernelGGL(mb_write3_bursts, dim3((uint32_t)((nq + 255) / 256)), dim3(64), lds, stream, P, M, V, nq, g_pattern); break;
        case 13: hipLaunchKernelGGL(mb_oneshot_x4, dim3((uint32_t)((nq + 255) / 256)), dim3(64), lds, stream, P, M, V, G, nq); break;
        case 14:
        case 15:
        case 16: {
            if (param < 0 || param > 24) return -1;
            const int64_t span = (int64_t)8 << param;
            const int64_t grid = (grid64 + span - 1) / span * span;  // whole groups: the surplus workgroups find no tile
            if (grid > 0x7ffffff0) return -1;
            if (kind == 14) hipLaunchKernelGGL(mb_oneshot_xcd, dim3((uint32_t)grid), dim3(64), lds, stream, P, M, V, G, nq, param);
            else if (kind == 15) hipLaunchKernelGGL(mb_memeff_both_xcd, dim3((uint32_t)grid), dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq, param);
            else hipLaunchKernelGGL(mb_write3_xcd, dim3((uint32_t)grid), dim3(64), lds, stream, P, M, V, nq, param, g_pattern);
            break;
        }
        case 17:
        case 18:
        case 19: {
            // param: the period in 10 ns ticks of the real-time counter; loads get the share of it that they have of the bytes
            if (param < 2 || param > 100000) return -1;
            const uint32_t period = (uint32_t)param, split = kind == 19 ? period * 12 / 22 : period * 16 / 28;
            if (kind == 17) hipLaunchKernelGGL(mb_oneshot_phased, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, G, nq, period, split);
            else if (kind == 18) hipLaunchKernelGGL(mb_oneshot_x4_phased, dim3((uint32_t)((nq + 255) / 256)), dim3(64), lds, stream, P, M, V, G, nq, period, split);
            else hipLaunchKernelGGL(mb_memeff_both_phased, dim3((uint32_t)grid64), dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq, period, split);
            break;
        }
        case 20:
        case 21:
        case 22: {
            // param: the policy bits (sc0 = 1, sc1 = 2, nt = 4) of the stores (20) or of the loads (21); the other side uses the builtin
            if (param < 0 || param > 7) return -1;
            const dim3 grid((uint32_t)grid64);
#define X(N, BITS)                                                                                                                               \
    if (param == N) {                                                                                                                            \
        if (kind == 20) hipLaunchKernelGGL((mb_memeff_both_policy<-1, N>), grid, dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq);          \
        else if (kind == 21) hipLaunchKernelGGL((mb_memeff_both_policy<N, -1>), grid, dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq);    \
        else hipLaunchKernelGGL((mb_memeff_both_policy<N, 6>), grid, dim3(64), lds, stream, (f2*)p, M, V, (const f2*)g, nq);                      \
    }
            MB_POLICY_CASES(X)
#undef X
            break;
        }
        case 28:
        case 23:
        case 24:
        case 25: {
            if (param < 0 || param > 7) return -1;
#define X(N, BITS)                                                                                                                               \
    if (param == N) {                                                                                                                            \
        if (kind == 28) hipLaunchKernelGGL(mb_write2_policy<N>, dim3((uint32_t)grid64), dim3(64), lds, stream, M, V, nq, g_pattern);                \
        else if (kind == 23) hipLaunchKernelGGL(mb_memeff_write_policy<N>, dim3((uint32_t)grid64), dim3(64), lds, stream, (f2*)p, M, V, nq, g_pattern); \
        else if (kind == 24) hipLaunchKernelGGL(mb_oneshot_policy<N>, dim3((uint32_t)grid64), dim3(64), lds, stream, P, M, V, G, nq);              \
        else hipLaunchKernelGGL(mb_oneshot_x4_policy<N>, dim3((uint32_t)((nq + 255) / 256)), dim3(64), lds, stream, P, M, V, G, nq);               \
    }
            MB_POLICY_CASES(X)
#undef X
            break;
        }
        case 29: {
            const int64_t n2 = numel / 2, grid = (n2 + 63) / 64;
            if (grid > 0x7ffffff0) return -1;
            hipLaunchKernelGGL(mb_memeff_half_tile, dim3((uint32_t)grid), dim3(64), lds, stream, (float*)p, (f2*)m, (f2*)v, (const float*)g, n2);
            break;
        }
        case 26: {
            // param: bits 0-2 store policy (4 = nt, 6 = sc1 nt), bits 4-7 log2 of the run per XCD, bits 8-9 log2 of the tiles per
            // wave (1, 2, 4), bit 12 workgroups of 256 threads
            const int policy = param & 7, log2_run = (param >> 4) & 15, log2_tiles = (param >> 8) & 3, wide = (param >> 12) & 1;
            if ((policy != 4 && policy != 6) || log2_tiles > 2) return -1;
            const int64_t per_group = (wide ? 256 : 64) << log2_tiles;
            int64_t grid = (nq + per_group - 1) / per_group;
            if (log2_run) { const int64_t span = (int64_t)8 << log2_run; grid = (grid + span - 1) / span * span; }
            if (grid > 0x7ffffff0) return -1;
#define LAB(P, T, B)                                                                                                                    \
    if (policy == P && (1 << log2_tiles) == T && (wide ? 256 : 64) == B)                                                                \
        hipLaunchKernelGGL((mb_memeff_lab<P, T, B>), dim3((uint32_t)grid), dim3(B), lds, stream, (f2*)p, M, V, (const f2*)g, nq, log2_run);
            LAB(4, 1, 64) LAB(4, 2, 64) LAB(4, 4, 64) LAB(4, 1, 256) LAB(4, 2, 256) LAB(4, 4, 256)
            LAB(6, 1, 64) LAB(6, 2, 64) LAB(6, 4, 64) LAB(6, 1, 256) LAB(6, 2, 256) LAB(6, 4, 256)
#undef LAB
            break;
        }
        default: return -1;
    }
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

// A plain 128-bit copy of known traffic (nbytes read + nbytes written), one wave64 per workgroup: what the profiler's
// FETCH_SIZE / WRITE_SIZE counters are scaled by (bench.py --calib-copy-bytes).  nbytes must be a multiple of 16 and both
// pointers 16-byte aligned.  Returns 0, -1 for a bad argument, -2 for a launch error.
int fsadam_membench_copy(void* dst, const void* src, int64_t nbytes, void* stream_) {
    if (!dst || !src || nbytes < 0 || (nbytes & 15) || ((uintptr_t)dst & 15) || ((uintptr_t)src & 15)) return -1;
    if (nbytes == 0) return 0;
    const int64_t quads = nbytes / 16, grid = (quads + 63) / 64;
    if (grid > 0x7fffffff) return -1;
    hipLaunchKernelGGL(mb_copy, dim3((uint32_t)grid), dim3(64), 20480, static_cast<hipStream_t>(stream_), (f4*)dst, (const f4*)src, quads);
    return hipGetLastError() == hipSuccess ? 0 : -2;
}

}  // extern "C"
