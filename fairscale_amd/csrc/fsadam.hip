// Fused multi-tensor Adam step for MI355X (gfx950): host code and C ABI (include/fsadam.h); the kernels
// are in adam_kernels.h and grad_kernels.h, what both sides share in fsadam_common.h.
//
// Takes the place of fairscale's one native module:
//   fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu   (update equations :94-130, step size :153-162,
//                                                                dtype dispatch :172-256)
//   fairscale/clib/fused_adam_cuda/multi_tensor_apply.cuh      (tensor-list launcher :40-130)
//
// Design.  The path is elementwise and HBM-bound (14-28 bytes per element against a few dozen
// flops), so there is no MFMA here; what decides the speed is how the memory system is driven.
// Measured on this part, a streaming kernel is fastest when
//   * every workgroup is "one-shot": it handles one small tile (a few KiB per stream) and exits, so
//     that the hardware dispatcher hands out tiles in address order and the set of DRAM pages in
//     use at any moment stays small (grid-stride loops let workgroups drift apart and lose ~20 %);
//   * only 10-13 waves are resident per compute unit: enough bytes in flight to cover the latency,
//     few enough that the active address window stays tight.  Residency is capped by giving each
//     workgroup a block of LDS it never touches (LDS is the one launch-time resource that bounds
//     residency without costing registers or bandwidth);
//   * every load/store instruction of a wave covers one contiguous span (lane i next to lane i+1),
//     128 bits per lane for fp32 streams and 64 or 128 bits per lane for fp16 streams; loads carry
//     the non-temporal hint (nothing is re-read) and stores are written through the L2 at device
//     scope on top of it (store_through in fsadam_common.h: 2 points of the HBM rate).
// The tensor list becomes a device-resident table of 64-byte chunk descriptors (five pointers
// already advanced to the chunk, element count), uploaded once and reused every step.  Consecutive
// tensors that continue each other in every stream are laid out as one (build_runs).  A wave finds its work with one shift and one scalar load: descriptor = table[block >> k],
// tile = block & (2^k - 1).  Large tensors share one descriptor among 2^k tiles, middle-sized ones
// among 16, small ones get one descriptor per tile, each class placed after the one before, so ONE
// launch covers any number of tensors (the reference needs a launch per 36 tensors / 320 chunks
// because its table travels by value in the kernel arguments).  Ragged tiles (the end of a tensor)
// take an element-wise path with the same arithmetic; full tiles of a tensor whose streams are only element-aligned use the same vector
// instructions at odd addresses.
//
// Arithmetic is IEEE float32 exactly as written in the reference source: separate multiplies and
// adds (compiled with -ffp-contract=off), correctly rounded division and square root (hipcc's
// default for fp32), round-to-nearest-even conversions to fp16.  Dividing by a power-of-two scale
// is done as a multiplication by its exact reciprocal, which gives the same bits.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <string>
#include <vector>

#include "fsadam.h"

#include "fsadam_common.h"
#include "adam_kernels.h"
#include "grad_kernels.h"

// --------------------------------------------------------------------------------------------
// fsadam_grad_pass_noalloc: device memory the library never allocates
// --------------------------------------------------------------------------------------------
// The descriptor table and the partial results of a gradient pass for callers that cannot allocate: one
// array per GPU, part of the loaded code object, held until the process ends.  Layout: the table
// (FSADAM_NOALLOC_MAX_DESCRIPTORS rows of 64 bytes), then the partials of the tiles' workgroups
// (FSADAM_NOALLOC_MAX_WORKGROUPS, and 7 more because the slots are handed out in eights), of the second reduction
// stage (512) and the total (1), 16 bytes each, and 16 bytes that say which call owns the array (fsadam_put_descs).
// In host code the name below is only a handle for hipGetSymbolAddress: the device address is looked up
// once per device (scratch_on_current_device) and only that pointer is ever handed to a kernel.
constexpr size_t kScratchTableBytes = (size_t)FSADAM_NOALLOC_MAX_DESCRIPTORS * 64;
constexpr size_t kScratchPartials = (size_t)FSADAM_NOALLOC_MAX_WORKGROUPS + 7 + 512 + 1 + 1;  // 7: the slots are handed out in eights; the last 16 bytes: who owns the array
constexpr size_t kScratchBytes = kScratchTableBytes + kScratchPartials * 16;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

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
    int64_t lds_throttle = -1;  // bytes of untouched LDS per workgroup (0 = no cap, -1 = per-mode default)
    int64_t grad_items = 0;     // gradient pass: 16-byte vectors per lane (2, 4 or 8; 0 = by kind of pass)
    int64_t grad_lds_throttle = -1;  // gradient pass: LDS ballast per workgroup (-1 = by kind of pass)
    int64_t grad_waves = 0;         // gradient pass: tiles (waves) per workgroup, 1, 4 or 16; 0 = by kind of pass
    int64_t mid_tiles = 16;         // tiles that share a descriptor of a middle-sized tensor (a power of two up to 64; 0 = no such class)
    int64_t upload_stream = 1;      // 1: tables are copied to the device on a stream of the library's own
    int64_t align_heads = 1;        // 1: a tensor whose streams start off a cache line gives up a short head so that the rest starts on one
    int64_t merge_runs = 1;         // 1: consecutive tensors that continue each other in every stream are laid out as one
};

// Residency that measured fastest with one wave64 per workgroup, one vector per lane per stream and stores that
// are written through (store_through): about 36-40 KiB of loads in flight per compute unit, i.e. 10 waves of the
// 4 KiB-per-wave modes and 12 of the 3 KiB-per-wave ones.  The hardware hands out LDS in granules of 1280 bytes
// (a sweep in steps of 256 bytes changes the rate only at multiples of 1280), so a ballast of B bytes allows
// floor(128 / ceil(B / 1280)) workgroups per compute unit: 11 520 -> 14, 12 288 -> 12, 14 080 -> 11, 15 360 -> 10,
// 16 640 and 17 920 -> 9, 19 200 -> 8; 13 and 15 cannot be had.  One wave more or less costs 0.3-1.5 points, two
// cost 2-4.  The optimum hardly moves with the size of the list (swept from 1e7 to 6.7e9 elements in every mode):
// only the smallest lists like one step more residency, which is worth 1-2 points there.
int64_t default_lds_throttle(int mode, int64_t total_elems) {
    switch (mode) {
        case FSADAM_FULL_PRECISION:
        case FSADAM_FULL_PRECISION_FP16_COPY:
        case FSADAM_MIXED_PRECISION: return total_elems < 50000000 ? 14080 : 15360;
        case FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION: return total_elems < 500000000 ? 11520 : 12288;
        default: return total_elems < 50000000 ? 11520 : 12288;
    }
}
Options g_opt;
std::mutex g_mutex;        // guards g_opt
std::mutex g_cache_mutex;  // guards the fsadam_step table cache

bool valid_mode(int mode) { return mode >= FSADAM_FULL_PRECISION && mode <= FSADAM_FULL_PRECISION_FP16_COPY; }

int size_p(int mode) { return (mode == FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION || mode == FSADAM_PURE_FP16) ? 2 : 4; }
int size_s(int mode) { return mode == FSADAM_PURE_FP16 ? 2 : 4; }
int size_g(int mode) { return (mode == FSADAM_FULL_PRECISION || mode == FSADAM_FULL_PRECISION_FP16_COPY) ? 4 : 2; }

bool aligned_to(const void* ptr, uintptr_t bytes) { return (reinterpret_cast<uintptr_t>(ptr) & (bytes - 1)) == 0; }

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
        if (mode_has_copy(mode) && !r.p_copy)
            return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": this mode needs p_copy");
        // anything less than element alignment cannot be a tensor of that dtype
        if (!aligned_to(r.p, size_p(mode)) || !aligned_to(r.m, size_s(mode)) || !aligned_to(r.v, size_s(mode)) ||
            !aligned_to(r.g, size_g(mode)) || (mode_has_copy(mode) && !aligned_to(r.p_copy, 2)))
            return fail(FSADAM_EINVAL, "tensor " + std::to_string(t) + ": pointer not aligned to its element size");
    }
    return FSADAM_OK;
}

char* advance(const void* base, int64_t elems, int elem_size) {
    return const_cast<char*>(static_cast<const char*>(base)) + elems * elem_size;
}

// Every stream, `first` elements in, aligned to the kElems elements a lane moves per instruction.
bool row_vector_ok(const FsAdamTensor& r, int mode, int64_t first = 0) {
    const uintptr_t e = mode_elems(mode);
    return aligned_to(advance(r.p, first, size_p(mode)), e * size_p(mode)) && aligned_to(advance(r.m, first, size_s(mode)), e * size_s(mode)) &&
           aligned_to(advance(r.v, first, size_s(mode)), e * size_s(mode)) && aligned_to(advance(r.g, first, size_g(mode)), e * size_g(mode)) &&
           (!mode_has_copy(mode) || aligned_to(advance(r.p_copy, first, 2), e * 2));
}

// Where a tensor's streams start relative to cache lines decides how fast its tiles run: a wave moves
// 512 or 1024 contiguous bytes of a stream per instruction, and when those spans straddle 128-byte
// lines every line is touched by two instructions (partial-line writes, reads fetched twice): a list of
// views packed back to back measured 62-65 % of the HBM rate against 77-79 % for the same list on
// line boundaries.  A view cannot be moved, but its first few elements can be given to a short
// descriptor of their own, so that all the tiles behind it start where the streams are aligned.
// The head is chosen among the counts that bring one of the streams onto a 128-byte or 1024-byte
// boundary, by the bytes each stream moves per element times how far off it stays:
// nothing for a 1 KiB boundary, a little for a line boundary, most for anything else.
constexpr int64_t kHeadMinElems = 8192;  // shorter tensors are left alone: a head would add a workgroup to a handful
int64_t misalignment_cost(const void* ptr, int64_t first, int elem_size, int bytes_moved) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(advance(ptr, first, elem_size));
    const int64_t off = (a & 1023u) == 0 ? 0 : (a & 127u) == 0 ? 1 : (a & 15u) == 0 ? 5 : 6;
    return off * bytes_moved;
}
int64_t head_elems(const FsAdamTensor& r, int mode, const Options& opt) {
    if (!opt.align_heads || r.numel < kHeadMinElems) return 0;
    struct Stream { const void* ptr; int size, moved; };
    const Stream streams[5] = {{r.p, size_p(mode), 2 * size_p(mode)}, {r.m, size_s(mode), 2 * size_s(mode)}, {r.v, size_s(mode), 2 * size_s(mode)},
                               {r.g, size_g(mode), size_g(mode)}, {mode_has_copy(mode) ? r.p_copy : nullptr, 2, 2}};
    auto cost = [&](int64_t head) {
        int64_t c = 0;
        for (const Stream& st : streams)
            if (st.ptr) c += misalignment_cost(st.ptr, head, st.size, st.moved);
        return c;
    };
    int64_t best = 0, best_cost = cost(0);
    if (best_cost == 0) return 0;  // every stream on a 1 KiB boundary already
    int64_t tried[10];
    int n_tried = 0;
    for (const Stream& st : streams) {
        if (!st.ptr) continue;
        for (uintptr_t boundary : {uintptr_t(128), uintptr_t(1024)}) {
            const uintptr_t a = reinterpret_cast<uintptr_t>(st.ptr);
            const int64_t head = (int64_t)(((boundary - (a & (boundary - 1))) & (boundary - 1)) / st.size);
            bool seen = head == 0;  // streams that are off by the same amount propose the same heads
            for (int k = 0; k < n_tried && !seen; ++k) seen = tried[k] == head;
            if (seen) continue;
            tried[n_tried++] = head;
            const int64_t c = cost(head);
            if (c < best_cost || (c == best_cost && head < best)) { best = head; best_cost = c; }
        }
    }
    return best;
}

int64_t floor_pow2(int64_t x) {
    int64_t p = 1;
    while (p * 2 <= x) p *= 2;
    return p;
}
int log2_exact(int64_t x) {
    int k = 0;
    while ((int64_t(1) << k) < x) ++k;
    return k;
}

// How a tensor list is cut into descriptors for given options.
struct Layout {
    int64_t tile_elems = 0;
    int64_t large_chunk_elems = 0;
    int64_t mid_chunk_elems = 0;  // 0: no middle class
    int64_t n_runs = 0;  // rows after merging (fsadam: build_runs); the three classes below count these
    int64_t n_large = 0, n_mid = 0, n_small = 0, n_empty = 0;
    int64_t n_large_descs = 0, n_mid_descs = 0, n_small_descs = 0;
    int64_t total_elems = 0;
    int64_t n_vector = 0, n_scalar = 0;

    int64_t large_blocks() const { return n_large_descs * (large_chunk_elems / tile_elems); }
    int64_t mid_blocks() const { return mid_chunk_elems ? n_mid_descs * (mid_chunk_elems / tile_elems) : 0; }
    int64_t blocks() const { return tile_elems ? large_blocks() + mid_blocks() + n_small_descs : 0; }
    int64_t descs() const { return n_large_descs + n_mid_descs + n_small_descs; }
};

int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// What is left of a tensor behind its head goes to shared descriptors of large_chunk_elems (class 2), of
// mid_chunk_elems (class 3) or to one descriptor per tile (class 1).
enum { kClassSmall = 1, kClassLarge = 2, kClassMid = 3 };
int class_of(int64_t body, const Layout& L) {
    if (body >= kLargeThreshold) return kClassLarge;
    if (L.mid_chunk_elems > 0 && body >= L.mid_chunk_elems) return kClassMid;
    return kClassSmall;
}
// A middle class only where its chunks stay well under the size that makes a tensor large.
int64_t mid_chunk_for(int64_t tile_elems, int64_t mid_tiles) {
    const int64_t chunk = tile_elems * mid_tiles;
    return (mid_tiles > 1 && 2 * chunk <= kLargeThreshold) ? chunk : 0;
}
// The launch's view of a layout.
TileMap tile_map(const Layout& L) {
    TileMap map;
    map.log2_large = (uint32_t)log2_exact(L.large_chunk_elems / L.tile_elems);
    map.n_large_descs = (uint32_t)L.n_large_descs;
    map.n_large_blocks = (uint32_t)L.large_blocks();
    map.log2_mid = L.mid_chunk_elems ? (uint32_t)log2_exact(L.mid_chunk_elems / L.tile_elems) : 0u;
    map.n_mid_descs = (uint32_t)L.n_mid_descs;
    map.n_mid_blocks = (uint32_t)L.mid_blocks();
    return map;
}

// Row b starts, in every stream, at the element behind row a's last one.
bool continues(const FsAdamTensor& a, const FsAdamTensor& b, int mode) {
    return advance(a.p, a.numel, size_p(mode)) == b.p && advance(a.m, a.numel, size_s(mode)) == b.m &&
           advance(a.v, a.numel, size_s(mode)) == b.v && advance(a.g, a.numel, size_g(mode)) == b.g &&
           (!mode_has_copy(mode) || advance(a.p_copy, a.numel, 2) == b.p_copy);
}

// The list as the layout sees it: empty rows dropped and, with option merge_runs, every maximal sequence of
// consecutive rows that continue each other in all streams (parameters that are back-to-back views of one
// buffer, with gradients and state laid out the same way, as OSS's buckets make them: oss.py:630-659,
// param_bucket.py:62-90) replaced by ONE row over the whole sequence.  The update of an element does not
// depend on where its tile starts, so the results are the same bits; what changes is that a list of
// thousands of views becomes the few long runs a flat shard is.  run_of[t] (optional): index of the run
// row t went into, -1 for an empty row.
void build_runs(const FsAdamTensor* tensors, int64_t n, int mode, bool merge, std::vector<FsAdamTensor>& runs, std::vector<int64_t>* run_of) {
    runs.clear();
    if (run_of) run_of->assign((size_t)n, -1);
    const FsAdamTensor* last = nullptr;  // the row the current run ends with
    for (int64_t t = 0; t < n; ++t) {
        if (tensors[t].numel == 0) continue;
        if (merge && last && continues(*last, tensors[t], mode)) runs.back().numel += tensors[t].numel;
        else runs.push_back(tensors[t]);
        last = &tensors[t];
        if (run_of) (*run_of)[(size_t)t] = (int64_t)runs.size() - 1;
    }
}

// The head of every run, computed once per table (it is asked for three times on the way to one).
void compute_heads(const std::vector<FsAdamTensor>& runs, int mode, const Options& opt, std::vector<int64_t>& heads) {
    heads.resize(runs.size());
    for (size_t k = 0; k < runs.size(); ++k) heads[k] = head_elems(runs[k], mode, opt);
}

// `runs`: the rows build_runs made (none empty); `heads`: compute_heads of them.
Layout compute_layout(const std::vector<FsAdamTensor>& runs, const std::vector<int64_t>& heads, int mode, const Options& opt) {
    Layout L;
    L.tile_elems = kBlock * mode_elems(mode);
    L.mid_chunk_elems = mid_chunk_for(L.tile_elems, opt.mid_tiles);
    L.n_runs = (int64_t)runs.size();
    int64_t min_large = 0;
    for (size_t k = 0; k < runs.size(); ++k) {
        const FsAdamTensor& r = runs[k];
        L.total_elems += r.numel;
        const int64_t head = heads[k], body = r.numel - head;
        (row_vector_ok(r, mode, head) ? L.n_vector : L.n_scalar) += 1;
        const int cls = class_of(body, L);
        if (cls == kClassLarge) {
            L.n_large += 1;
            if (min_large == 0 || body < min_large) min_large = body;
        } else {
            (cls == kClassMid ? L.n_mid : L.n_small) += 1;
        }
    }
    // every large tensor spans at least two chunks ...
    L.large_chunk_elems = std::max(kMinLargeChunk, std::min(kMaxLargeChunk, floor_pow2(std::max<int64_t>(1, min_large / 2))));
    // ... and the tiles behind the tensors' ends (launched, find nothing to do, exit) stay under 1 % of all tiles: a
    // chunk that does not divide the tensors well is halved until they do (the Llama-7B list: 2^23 leaves the last
    // chunk of every 4096 x 11008 matrix 5/8 empty, 7 % of all workgroups; 2^20 divides every matrix of the list)
    for (; L.large_chunk_elems > kMinLargeChunk; L.large_chunk_elems /= 2) {
        int64_t body_total = 0, padded_total = 0;
        for (size_t k = 0; k < runs.size(); ++k) {
            const int64_t body = runs[k].numel - heads[k];
            if (class_of(body, L) != kClassLarge) continue;
            body_total += body;
            padded_total += ceil_div(body, L.large_chunk_elems) * L.large_chunk_elems;
        }
        if ((padded_total - body_total) * 100 <= body_total) break;
    }
    for (size_t k = 0; k < runs.size(); ++k) {
        const int64_t head = heads[k], body = runs[k].numel - head;
        L.n_small_descs += ceil_div(head, L.tile_elems);
        const int cls = class_of(body, L);
        if (cls == kClassLarge) L.n_large_descs += ceil_div(body, L.large_chunk_elems);
        else if (cls == kClassMid) L.n_mid_descs += ceil_div(body, L.mid_chunk_elems);
        else L.n_small_descs += ceil_div(body, L.tile_elems);
    }
    return L;
}

}  // namespace

// "Everything enqueued so far that uses X" as something a stream or the host can wait for.  By default
// the event is recorded right behind every use.  A plan that was told so (fsadam_plan_lazy_events) records it only when
// somebody needs it (another stream takes over, the table slot is about to be overwritten, the plan
// goes away), so that a step on the stream of the step before enqueues its kernel and nothing else
// (3 us less per step); recording late marks a later point of the same stream, which covers the uses
// as well, but it touches the stream after the call that used it has returned: the caller must then
// keep every stream it has passed to that plan alive for as long as the plan lives.
struct UseMark {
    hipEvent_t event = nullptr;
    hipStream_t stream = nullptr;  // where the uses were enqueued
    bool used = false;             // there has been a use
    bool pending = false;          // uses enqueued on `stream` since the event was last recorded
};

// A device table plus its pinned staging copy.  A plan keeps a small ring of them: when a pointer
// of the list moves, the new table goes into the next slot, so the host only ever waits for the
// step that used that slot kTableSlots updates ago, not for the step still in flight.
struct TableSlot {
    int64_t cap_descs = 0;
    ChunkDesc* d_table = nullptr;
    ChunkDesc* h_table = nullptr;  // pinned, or ordinary host memory for a table short enough to travel in kernel arguments
    bool pinned = false;
    UseMark mark;
    hipEvent_t uploaded = nullptr;  // the copy of h_table into d_table, when it went over the library's own stream
};
constexpr int kTableSlots = 3;

struct FsAdamPlan {
    int mode = 0;
    int device = -1;
    hipStream_t upload_stream = nullptr;  // the library's own, for tables (see upload_table)
    Options opt;                     // as asked for when the table was set (lds_throttle may be -1: by mode and size)
    int64_t lds_bytes = 0;           // the ballast the current table is stepped with
    Layout layout;
    std::vector<FsAdamTensor> rows;  // what the current table was built from
    std::vector<FsAdamTensor> runs;  // scratch of plan_set_tensors: the rows after merging
    std::vector<int64_t> heads;      // ... and the head of each
    bool lazy_events = false;        // see UseMark; fsadam_plan_lazy_events
    int64_t uploads = 0;
    TableSlot slots[kTableSlots];
    int current = -1;  // slot holding the table of `rows`
    uint64_t lru = 0;  // fsadam_step cache bookkeeping
};

namespace {

int mark_init(UseMark& m) {
    if (!m.event) FS_HIP(hipEventCreateWithFlags(&m.event, hipEventDisableTiming));
    return FSADAM_OK;
}
// A use has been enqueued on `stream` (after mark_order_after for that stream).
int mark_use(UseMark& m, hipStream_t stream, bool lazy) {
    m.stream = stream;
    m.used = true;
    m.pending = lazy;
    if (!lazy) FS_HIP(hipEventRecord(m.event, stream));
    return FSADAM_OK;
}
// Make the event cover every use enqueued so far.  A stream that cannot take the record any more (the
// caller destroyed it) has nothing left in flight that a device-wide wait would not cover.
int mark_settle(UseMark& m) {
    if (!m.pending) return FSADAM_OK;
    if (hipEventRecord(m.event, m.stream) != hipSuccess) {
        (void)hipGetLastError();
        FS_HIP(hipDeviceSynchronize());
        m.used = false;
    }
    m.pending = false;
    return FSADAM_OK;
}
// The host waits until every use has finished.
int mark_wait(UseMark& m) {
    const int rc = mark_settle(m);
    if (rc) return rc;
    if (m.used && m.event) FS_HIP(hipEventSynchronize(m.event));
    return FSADAM_OK;
}
// Work about to be enqueued on `stream` is ordered after the uses so far when the caller has moved to
// another stream; on one stream the order is already there.
int mark_order_after(UseMark& m, hipStream_t stream) {
    if (!m.used || m.stream == stream) return FSADAM_OK;
    const int rc = mark_settle(m);
    if (rc) return rc;
    if (m.used) FS_HIP(hipStreamWaitEvent(stream, m.event, 0));
    return FSADAM_OK;
}
void mark_destroy(UseMark& m) {
    (void)mark_wait(m);
    if (m.event) (void)hipEventDestroy(m.event);
    m = UseMark();
}

// A new table is copied to the device on a stream of the library's own and the caller's stream only waits
// for that copy's event: the copy (1.4 MB for a 4096-tensor list, 60 us) then runs while the step before
// is still busy on the caller's stream instead of between the two steps.  `own_stream` = 0 (option
// "upload_stream") puts the copy on the caller's stream.
int upload_table(hipStream_t* own, bool use_own, TableSlot& slot, int64_t n_descs, hipStream_t stream) {
    if (n_descs <= 0) return FSADAM_OK;
    if (n_descs <= kDescsPerPut) {
        // A table this short (a flat shard under 8e8 elements, a handful of tensors) travels in the arguments of one small
        // launch on the caller's stream, in front of the step that reads it: no copy engine, no second stream, no event.
        // For a one-tensor list whose gradient is another tensor every step that halves what a step costs (60 -> 35 us).
        DescBatch batch;
        std::memcpy(batch.rows, slot.h_table, (size_t)n_descs * sizeof(ChunkDesc));
        hipLaunchKernelGGL(fsadam_put_descs, dim3(1), dim3(64), 0, stream, slot.d_table, batch, 0u, (uint32_t)n_descs, (uint32_t*)nullptr, 0u);
        FS_HIP(hipGetLastError());
        return FSADAM_OK;
    }
    const size_t bytes = (size_t)n_descs * sizeof(ChunkDesc);
    if (!use_own) {
        FS_HIP(hipMemcpyAsync(slot.d_table, slot.h_table, bytes, hipMemcpyHostToDevice, stream));
        return FSADAM_OK;
    }
    if (!*own) FS_HIP(hipStreamCreateWithFlags(own, hipStreamNonBlocking));
    if (!slot.uploaded) FS_HIP(hipEventCreateWithFlags(&slot.uploaded, hipEventDisableTiming));
    FS_HIP(hipMemcpyAsync(slot.d_table, slot.h_table, bytes, hipMemcpyHostToDevice, *own));
    FS_HIP(hipEventRecord(slot.uploaded, *own));
    FS_HIP(hipStreamWaitEvent(stream, slot.uploaded, 0));
    return FSADAM_OK;
}
void upload_stream_destroy(hipStream_t* own) {
    if (!*own) return;
    (void)hipStreamSynchronize(*own);
    (void)hipStreamDestroy(*own);
    *own = nullptr;
}

void slot_release(TableSlot& slot) {
    (void)mark_wait(slot.mark);
    if (slot.d_table) (void)hipFree(slot.d_table);
    if (slot.h_table) {
        if (slot.pinned) (void)hipHostFree(slot.h_table);
        else std::free(slot.h_table);
    }
    slot.d_table = slot.h_table = nullptr;
    slot.cap_descs = 0;
    slot.pinned = false;
    slot.mark.used = slot.mark.pending = false;
}

// Room for a table of n_descs rows in a slot nothing reads any more.  A table short enough to travel in kernel arguments
// (upload_table) is staged in ordinary host memory: pinning a page costs 35-140 us, which is most of what the first
// steps of a small list would spend.
int slot_reserve(TableSlot& slot, int64_t n_descs) {
    const bool want_pinned = n_descs > kDescsPerPut;
    if (n_descs <= slot.cap_descs && (slot.pinned || !want_pinned)) return FSADAM_OK;
    slot_release(slot);
    const int64_t cap = want_pinned ? std::max<int64_t>(n_descs + n_descs / 8, 64) : kDescsPerPut;
    if (hipMalloc(reinterpret_cast<void**>(&slot.d_table), cap * sizeof(ChunkDesc)) != hipSuccess) {
        slot.d_table = nullptr;
        return fail(FSADAM_ENOMEM, "hipMalloc of the descriptor table failed");
    }
    if (want_pinned) {
        if (hipHostMalloc(reinterpret_cast<void**>(&slot.h_table), cap * sizeof(ChunkDesc), hipHostMallocDefault) != hipSuccess) slot.h_table = nullptr;
    } else {
        slot.h_table = static_cast<ChunkDesc*>(std::malloc((size_t)cap * sizeof(ChunkDesc)));
    }
    if (!slot.h_table) {
        (void)hipFree(slot.d_table);
        slot.d_table = nullptr;
        return fail(FSADAM_ENOMEM, "allocation of the descriptor staging buffer failed");
    }
    slot.pinned = want_pinned;
    slot.cap_descs = cap;
    return FSADAM_OK;
}

// The scalars of a step (step size, scales) travel by value in the kernel arguments and the table slots
// are guarded by events the host waits on: recorded into a HIP graph, every replay would repeat the
// first step's bias correction and the events could never be waited for.  Refuse instead of going wrong.
int refuse_capture(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    FS_HIP(hipStreamIsCapturing(stream, &status));
    if (status != hipStreamCaptureStatusNone)
        return fail(FSADAM_EINVAL, "the stream is being captured into a graph: this call cannot be recorded (its step-dependent scalars are kernel arguments)");
    return FSADAM_OK;
}

// events and streams belong to the device they were created on: they go with the buffers
void slot_destroy(TableSlot& slot) {
    slot_release(slot);
    mark_destroy(slot.mark);
    if (slot.uploaded) (void)hipEventDestroy(slot.uploaded);
    slot.uploaded = nullptr;
}

void plan_release_buffers(FsAdamPlan* plan) {
    for (TableSlot& slot : plan->slots) slot_destroy(slot);
    upload_stream_destroy(&plan->upload_stream);
    plan->current = -1;
}

// Descriptors for elements [start, start + count) of a tensor, chunk_elems each; returns how many.
int64_t fill_descs(ChunkDesc* out, const FsAdamTensor& r, int mode, int64_t start, int64_t count, int64_t chunk_elems) {
    const int64_t chunks = ceil_div(count, chunk_elems);
    for (int64_t c = 0; c < chunks; ++c) {
        const int64_t first = start + c * chunk_elems;
        ChunkDesc& d = out[c];
        d.p = advance(r.p, first, size_p(mode));
        d.m = advance(r.m, first, size_s(mode));
        d.v = advance(r.v, first, size_s(mode));
        d.g = advance(r.g, first, size_g(mode));
        d.p_copy = mode_has_copy(mode) ? advance(r.p_copy, first, 2) : nullptr;
        d.n = (uint32_t)std::min<int64_t>(chunk_elems, start + count - first);
        d.pad32 = 0;
        d.pad = 0;
    }
    return chunks;
}

template <int MODE>
int launch_tiles(const ChunkDesc* table, const Layout& L, int64_t lds_bytes, const StepScalars& s, float* found_inf, hipStream_t stream) {
    const int64_t n_blocks = L.blocks();
    if (n_blocks == 0) return FSADAM_OK;
    if (n_blocks > 0x7ffffff0) return fail(FSADAM_EINVAL, "tensor list too large for one launch");
    hipLaunchKernelGGL((fsadam_tiles<MODE, kBlock, 1>), dim3((uint32_t)n_blocks), dim3(kBlock), (size_t)lds_bytes, stream, table, tile_map(L), s,
                       found_inf);
    FS_HIP(hipGetLastError());
    return FSADAM_OK;
}

int launch_mode(int mode, const ChunkDesc* table, const Layout& L, int64_t lds_bytes, const StepScalars& s, float* found_inf,
                hipStream_t stream) {
#define FS_MODE(M) \
    case M: return launch_tiles<M>(table, L, lds_bytes, s, found_inf, stream)
    switch (mode) {
        FS_MODE(FSADAM_FULL_PRECISION);
        FS_MODE(FSADAM_MIXED_PRECISION);
        FS_MODE(FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION);
        FS_MODE(FSADAM_FULL_PRECISION_FP16_COPY);
        default: return launch_tiles<FSADAM_PURE_FP16>(table, L, lds_bytes, s, found_inf, stream);
    }
#undef FS_MODE
}

// A list that does not pass validation changes nothing.  A failure later on (an allocation, a HIP call) leaves the
// plan without tensors (plan_step refuses) rather than with a layout that does not belong to the table on the device.
int plan_set_tensors(FsAdamPlan* plan, const FsAdamTensor* tensors, int64_t n, hipStream_t stream) {
    // a list that is refused outright leaves the plan with the table it had
    int rc = validate_rows(tensors, n, plan->mode);
    if (rc) return rc;
    rc = refuse_capture(stream);
    if (rc) return rc;
    plan->rows.clear();  // from here on a failure leaves the plan without tensors
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (plan->device != dev) {
        plan_release_buffers(plan);
        plan->device = dev;
    }
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        plan->opt = g_opt;
    }
    build_runs(tensors, n, plan->mode, plan->opt.merge_runs != 0, plan->runs, nullptr);
    compute_heads(plan->runs, plan->mode, plan->opt, plan->heads);
    Layout L = compute_layout(plan->runs, plan->heads, plan->mode, plan->opt);
    for (int64_t t = 0; t < n; ++t) L.n_empty += tensors[t].numel == 0 ? 1 : 0;
    const int64_t lds_bytes = plan->opt.lds_throttle >= 0 ? plan->opt.lds_throttle : default_lds_throttle(plan->mode, L.total_elems);
    const int64_t n_descs = L.descs();
    if (L.blocks() > 0x7ffffff0) return fail(FSADAM_EINVAL, "tensor list too large for one launch");

    // next slot of the ring; it may still be read by the step that used it last
    TableSlot& slot = plan->slots[(plan->current + 1) % kTableSlots];
    rc = mark_init(slot.mark);
    if (rc) return rc;
    rc = mark_wait(slot.mark);
    if (rc) return rc;
    rc = slot_reserve(slot, n_descs);
    if (rc) return rc;
    // descriptors of large tensors first, then the middle-sized ones, then one per tile: one launch covers all
    ChunkDesc* large = slot.h_table;
    ChunkDesc* mid = large + L.n_large_descs;
    ChunkDesc* small = mid + L.n_mid_descs;
    for (size_t k = 0; k < plan->runs.size(); ++k) {
        const FsAdamTensor& r = plan->runs[k];
        const int64_t head = plan->heads[k], body = r.numel - head;
        small += fill_descs(small, r, plan->mode, 0, head, L.tile_elems);
        const int cls = class_of(body, L);
        if (cls == kClassLarge) large += fill_descs(large, r, plan->mode, head, body, L.large_chunk_elems);
        else if (cls == kClassMid) mid += fill_descs(mid, r, plan->mode, head, body, L.mid_chunk_elems);
        else small += fill_descs(small, r, plan->mode, head, body, L.tile_elems);
    }
    if (large != slot.h_table + L.n_large_descs || mid != slot.h_table + L.n_large_descs + L.n_mid_descs || small != slot.h_table + n_descs)
        return fail(FSADAM_EINVAL, "internal error: descriptor count differs from the layout");
    rc = upload_table(&plan->upload_stream, plan->opt.upload_stream != 0, slot, n_descs, stream);
    if (rc) return rc;
    rc = mark_use(slot.mark, stream, plan->lazy_events);
    if (rc) return rc;
    // the steps that used the table this one replaces are all enqueued: their slot's event can be taken now
    if (plan->current >= 0) {
        rc = mark_settle(plan->slots[plan->current].mark);
        if (rc) return rc;
    }
    // everything went through: the plan now describes the new table
    plan->layout = L;
    plan->lds_bytes = lds_bytes;
    plan->rows.assign(tensors, tensors + n);
    plan->current = (plan->current + 1) % kTableSlots;
    plan->uploads += 1;
    return FSADAM_OK;
}

int plan_step(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, float grad_scale, const float* grad_scale_dev,
              float optim_scale, float decay, int step, int eps_mode, int bias_correction, float* found_inf, hipStream_t stream) {
    if (plan->rows.empty() || plan->current < 0) return fail(FSADAM_EINVAL, "plan has no tensors; call fsadam_plan_set_tensors first");
    if (eps_mode != FSADAM_EPS_INSIDE_SQRT && eps_mode != FSADAM_EPS_OUTSIDE_SQRT)
        return fail(FSADAM_EINVAL, "eps_mode must be 0 (inside sqrt) or 1 (outside)");
    if (plan->mode == FSADAM_PURE_FP16 && !found_inf) return fail(FSADAM_EINVAL, "PURE_FP16 needs a found_inf device pointer");
    if (int refused = refuse_capture(stream)) return refused;
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(FSADAM_EINVAL, "plan belongs to device " + std::to_string(plan->device) + ", current device is " + std::to_string(dev));

    StepScalars s;
    s.b1 = beta1; s.b2 = beta2;
    s.one_minus_b1 = 1 - beta1;  // float subtraction as in the device code of the reference (kernel.cu:97,118)
    s.one_minus_b2 = 1 - beta2;
    s.eps = eps; s.decay = decay;
    s.step_size = fsadam_step_size(lr, beta1, beta2, step, bias_correction);
    s.grad_scale = grad_scale; s.optim_scale = optim_scale;
    s.inv_grad_scale = 0.f; s.inv_optim_scale = 0.f;
    s.eps_mode = eps_mode;
    s.grad_scale_dev = grad_scale_dev;
    const bool gs_ok = grad_scale_dev == nullptr && is_pow2_with_exact_reciprocal(grad_scale, &s.inv_grad_scale);
    const bool os_ok = is_pow2_with_exact_reciprocal(optim_scale, &s.inv_optim_scale);
    s.fast_scales = (gs_ok && (plan->mode != FSADAM_PURE_FP16 || os_ok)) ? 1 : 0;

    const Layout& L = plan->layout;
    TableSlot& slot = plan->slots[plan->current];
    int rc = mark_order_after(slot.mark, stream);
    if (rc) return rc;
    rc = launch_mode(plan->mode, slot.d_table, L, plan->lds_bytes, s, found_inf, stream);
    if (rc) return rc;
    return mark_use(slot.mark, stream, plan->lazy_events);
}

// m = v = 0 for every tensor of the plan's current table: one launch over the step's own layout.
int plan_zero_state(FsAdamPlan* plan, hipStream_t stream) {
    if (plan->rows.empty() || plan->current < 0) return fail(FSADAM_EINVAL, "plan has no tensors; call fsadam_plan_set_tensors first");
    if (int refused = refuse_capture(stream)) return refused;
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (dev != plan->device)
        return fail(FSADAM_EINVAL, "plan belongs to device " + std::to_string(plan->device) + ", current device is " + std::to_string(dev));
    const Layout& L = plan->layout;
    const int64_t n_blocks = L.blocks();
    if (n_blocks == 0) return FSADAM_OK;
    TableSlot& slot = plan->slots[plan->current];
    int rc = mark_order_after(slot.mark, stream);
    if (rc) return rc;
    // a pass that only writes through runs best with 10-13 waves per compute unit: 95-96 % of the HBM rate at 12-16 KiB of
    // ballast, 85-90 % at 8 or 20 KiB, under 50 % from 32 KiB on (a wave's stores are acknowledged by the memory, not the L2)
    const size_t lds = 14336;
    if (plan->mode == FSADAM_PURE_FP16)
        hipLaunchKernelGGL((fsadam_zero_state<FSADAM_PURE_FP16, kBlock>), dim3((uint32_t)n_blocks), dim3(kBlock), lds, stream, slot.d_table, tile_map(L));
    else
        hipLaunchKernelGGL((fsadam_zero_state<FSADAM_FULL_PRECISION, kBlock>), dim3((uint32_t)n_blocks), dim3(kBlock), lds, stream, slot.d_table, tile_map(L));
    FS_HIP(hipGetLastError());
    return mark_use(slot.mark, stream, plan->lazy_events);
}


// ---- gradient pass, host side -----------------------------------------------------------------

struct GradPlan {
    int device = -1;
    int dtype = 0;
    int64_t items = 4;
    int64_t lds_throttle = 0;
    int64_t align_heads = 1;
    int64_t mid_tiles = 16;
    bool own_upload_stream = true;
    hipStream_t upload_stream = nullptr;
    int64_t waves = 1;  // tiles per workgroup: 1, 4 or 16
    std::vector<FsGradTensor> rows;
    Layout layout;
    TableSlot slots[kTableSlots];
    int current = -1;
    GradPartial* d_partials = nullptr;  // [cap_partials] first stage, then [kReduceBlocks] second stage, then [1] total
    int64_t cap_partials = 0;
    UseMark partials_mark;  // the partial sums are shared by every call of the plan
    uint64_t lru = 0;
};

constexpr int kReduceBlocks = 512;
constexpr int kSlotSlack = 7;  // the partials of n workgroups take 8 * ceil(n / 8) slots

int grad_elem_size(int dtype) { return dtype == FSADAM_GRAD_F16 ? 2 : 4; }
int64_t grad_tile_elems(int dtype, int64_t items) { return 64 * (16 / grad_elem_size(dtype)) * items; }

// The one stream of the gradient pass: the elements in front of the next 1 KiB boundary go to a
// descriptor of their own, as in the step.
int64_t grad_head_elems(const FsGradTensor& r, int elem_size, int64_t align_heads) {
    if (!align_heads || r.numel < kHeadMinElems) return 0;
    const uintptr_t a = reinterpret_cast<uintptr_t>(r.g);
    return (int64_t)(((1024 - (a & 1023u)) & 1023u) / (uintptr_t)elem_size);
}

Layout grad_layout(const FsGradTensor* grads, int64_t n, int dtype, int64_t items, int64_t align_heads, int64_t mid_tiles) {
    Layout L;
    L.tile_elems = grad_tile_elems(dtype, items);
    L.mid_chunk_elems = mid_chunk_for(L.tile_elems, mid_tiles);
    const int esz = grad_elem_size(dtype);
    int64_t min_large = 0;
    for (int64_t t = 0; t < n; ++t) {
        const int64_t numel = grads[t].numel;
        L.total_elems += numel;
        if (numel == 0) { L.n_empty += 1; continue; }
        const int64_t head = grad_head_elems(grads[t], esz, align_heads), body = numel - head;
        (aligned_to(advance(grads[t].g, head, esz), 16) ? L.n_vector : L.n_scalar) += 1;
        const int cls = class_of(body, L);
        if (cls == kClassLarge) {
            L.n_large += 1;
            if (min_large == 0 || body < min_large) min_large = body;
        } else {
            (cls == kClassMid ? L.n_mid : L.n_small) += 1;
        }
    }
    L.large_chunk_elems = std::max(kMinLargeChunk, std::min(kMaxLargeChunk, floor_pow2(std::max<int64_t>(1, min_large / 2))));
    for (; L.large_chunk_elems > kMinLargeChunk; L.large_chunk_elems /= 2) {  // tiles behind the tensors' ends under 1 %, as in compute_layout
        int64_t body_total = 0, padded_total = 0;
        for (int64_t t = 0; t < n; ++t) {
            if (grads[t].numel == 0) continue;
            const int64_t body = grads[t].numel - grad_head_elems(grads[t], esz, align_heads);
            if (class_of(body, L) != kClassLarge) continue;
            body_total += body;
            padded_total += ceil_div(body, L.large_chunk_elems) * L.large_chunk_elems;
        }
        if ((padded_total - body_total) * 100 <= body_total) break;
    }
    for (int64_t t = 0; t < n; ++t) {
        const int64_t numel = grads[t].numel;
        if (numel == 0) continue;
        const int64_t head = grad_head_elems(grads[t], esz, align_heads), body = numel - head;
        L.n_small_descs += ceil_div(head, L.tile_elems);
        const int cls = class_of(body, L);
        if (cls == kClassLarge) L.n_large_descs += ceil_div(body, L.large_chunk_elems);
        else if (cls == kClassMid) L.n_mid_descs += ceil_div(body, L.mid_chunk_elems);
        else L.n_small_descs += ceil_div(body, L.tile_elems);
    }
    return L;
}

// The descriptors of a gradient list under layout L, written to table[0 .. L.descs()): large tensors first,
// then the middle-sized ones, then one per tile.  False when the count does not come out as L says.
bool grad_fill_table(ChunkDesc* table, const Layout& L, const FsGradTensor* grads, int64_t n, int esz, int64_t align_heads) {
    ChunkDesc* large = table;
    ChunkDesc* mid = large + L.n_large_descs;
    ChunkDesc* small = mid + L.n_mid_descs;
    for (int64_t t = 0; t < n; ++t) {
        const FsGradTensor& r = grads[t];
        if (r.numel == 0) continue;
        const int64_t head = grad_head_elems(r, esz, align_heads);
        // pieces: the head (tile-sized descriptors), then the rest in shared chunks or tiles
        const struct { int64_t start, count; int cls; } pieces[2] = {{0, head, kClassSmall}, {head, r.numel - head, class_of(r.numel - head, L)}};
        for (const auto& piece : pieces) {
            const int64_t chunk_elems = piece.cls == kClassLarge ? L.large_chunk_elems : piece.cls == kClassMid ? L.mid_chunk_elems : L.tile_elems;
            const int64_t chunks = ceil_div(piece.count, chunk_elems);
            ChunkDesc*& out = piece.cls == kClassLarge ? large : piece.cls == kClassMid ? mid : small;
            for (int64_t c = 0; c < chunks; ++c) {
                ChunkDesc& d = out[c];
                std::memset(&d, 0, sizeof(d));
                const int64_t first = piece.start + c * chunk_elems;
                d.g = advance(r.g, first, esz);
                d.n = (uint32_t)std::min<int64_t>(chunk_elems, piece.start + piece.count - first);
            }
            out += chunks;
        }
    }
    return large == table + L.n_large_descs && mid == table + L.n_large_descs + L.n_mid_descs && small == table + L.descs();
}

void grad_plan_free(GradPlan* plan) {
    mark_destroy(plan->partials_mark);
    for (TableSlot& slot : plan->slots) slot_destroy(slot);
    upload_stream_destroy(&plan->upload_stream);
    if (plan->d_partials) (void)hipFree(plan->d_partials);
    delete plan;
}

// Measured best shapes, one wave per workgroup either way (consecutive tiles then run on different XCDs, which
// the memory channels like best): a pass that only reads takes 8 vectors per lane (8 KiB per wave) at 11 waves per
// compute unit, a pass that writes the gradients back 4 vectors at 12 waves, like the Adam kernels.
void grad_shape(bool writes, int64_t* items, int64_t* lds, int64_t* waves, int64_t* align_heads, int64_t* mid_tiles, int64_t* upload_stream) {
    std::lock_guard<std::mutex> lock(g_mutex);
    *upload_stream = g_opt.upload_stream;
    *mid_tiles = g_opt.mid_tiles;
    *align_heads = g_opt.align_heads;
    *waves = g_opt.grad_waves ? g_opt.grad_waves : 1;
    *items = g_opt.grad_items ? g_opt.grad_items : (writes ? 4 : 8);
    *lds = g_opt.grad_lds_throttle >= 0 ? g_opt.grad_lds_throttle : (writes ? 12800 : 14080);
}

int grad_plan_set(GradPlan* plan, const FsGradTensor* grads, int64_t n, hipStream_t stream) {
    const Layout L = grad_layout(grads, n, plan->dtype, plan->items, plan->align_heads, plan->mid_tiles);
    const int64_t n_blocks = L.blocks();
    if (n_blocks > 0x7ffffff0) return fail(FSADAM_EINVAL, "gradient list too large for one launch");
    const int64_t n_descs = L.descs();
    TableSlot& slot = plan->slots[(plan->current + 1) % kTableSlots];
    int rc = mark_init(slot.mark);
    if (rc) return rc;
    rc = mark_init(plan->partials_mark);
    if (rc) return rc;
    rc = mark_wait(slot.mark);
    if (rc) return rc;
    rc = slot_reserve(slot, n_descs);
    if (rc) return rc;
    if (n_blocks + kSlotSlack + kReduceBlocks + 1 > plan->cap_partials) {
        // the partials may still be read by the reduction of the previous call
        rc = mark_wait(plan->partials_mark);
        if (rc) return rc;
        if (plan->d_partials) (void)hipFree(plan->d_partials);
        plan->d_partials = nullptr;
        plan->cap_partials = 0;
        const int64_t cap = n_blocks + kSlotSlack + n_blocks / 8 + kReduceBlocks + 1;
        if (hipMalloc(reinterpret_cast<void**>(&plan->d_partials), cap * sizeof(GradPartial)) != hipSuccess) {
            plan->d_partials = nullptr;
            return fail(FSADAM_ENOMEM, "hipMalloc of the partial sums failed");
        }
        plan->cap_partials = cap;
    }
    if (!grad_fill_table(slot.h_table, L, grads, n, grad_elem_size(plan->dtype), plan->align_heads))
        return fail(FSADAM_EINVAL, "internal error: descriptor count differs from the layout");
    plan->layout = L;
    plan->rows.assign(grads, grads + n);
    rc = upload_table(&plan->upload_stream, plan->own_upload_stream, slot, n_descs, stream);
    if (rc) return rc;
    rc = mark_use(slot.mark, stream, false);
    if (rc) return rc;
    if (plan->current >= 0) {
        rc = mark_settle(plan->slots[plan->current].mark);
        if (rc) return rc;
    }
    plan->current = (plan->current + 1) % kTableSlots;
    return FSADAM_OK;
}

// The launches of one pass: the tiles (workgroups of `waves` consecutive tiles, one partial each, into
// first[0 .. n_groups)), then two fixed-shape reduction steps through second[0 .. kReduceBlocks) and total[0],
// the last of which publishes.  Shared by fsadam_grad_pass and its variant that allocates nothing.
template <typename T>
int grad_launch(const ChunkDesc* table, const Layout& L, int64_t waves, int64_t items, size_t lds, float inv_scale, const float* inv_scale_dev,
                int write_back, GradPartial* first, GradPartial* second, GradPartial* total, float* found_inf, double* sum_squares,
                float* abs_max, hipStream_t stream, uint32_t* owner = nullptr, uint32_t ticket = 0) {
    const int64_t n_blocks = L.blocks();
    const TileMap map = tile_map(L);
    const int64_t n_groups = ceil_div(n_blocks, waves);
    // the workgroups' partials lie in 8 rows of per_xcd slots (see fsadam_grad_tiles): n_slots <= n_groups + kSlotSlack
    const uint32_t per_xcd = (uint32_t)ceil_div(std::max<int64_t>(n_groups, 1), 8);
    const int64_t n_slots = (int64_t)per_xcd * 8;
#define FS_GRAD_LAUNCH(WAVES, ITEMS)                                                                                          \
    hipLaunchKernelGGL((fsadam_grad_tiles<T, WAVES, ITEMS>), dim3((uint32_t)n_groups), dim3(64 * WAVES), lds, stream,        \
                       table, map, (uint32_t)n_blocks, inv_scale, inv_scale_dev, write_back, first, per_xcd)
#define FS_GRAD_ITEMS(WAVES)                          \
    do {                                              \
        if (items == 2) FS_GRAD_LAUNCH(WAVES, 2);      \
        else if (items == 8) FS_GRAD_LAUNCH(WAVES, 8); \
        else FS_GRAD_LAUNCH(WAVES, 4);                 \
    } while (0)
    if (n_blocks > 0) {
        if (waves == 16) FS_GRAD_ITEMS(16);
        else if (waves == 4) FS_GRAD_ITEMS(4);
        else FS_GRAD_ITEMS(1);
    }
#undef FS_GRAD_ITEMS
#undef FS_GRAD_LAUNCH
    FS_HIP(hipGetLastError());
    // two fixed-shape reduction steps, the second of which publishes (also when the list holds no element: everything is zero)
    const uint32_t blocks2 = (uint32_t)std::max<int64_t>(1, std::min<int64_t>(kReduceBlocks, ceil_div(n_slots, 1024)));
    const uint32_t per_block = (uint32_t)ceil_div(n_slots, blocks2);
    hipLaunchKernelGGL(fsadam_grad_reduce, dim3(blocks2), dim3(256), 0, stream, first, (uint32_t)n_slots, per_block, second, 0, 0,
                       (float*)nullptr, (double*)nullptr, (float*)nullptr, per_xcd, (uint32_t)n_groups, (uint32_t*)nullptr, 0u);
    hipLaunchKernelGGL(fsadam_grad_reduce, dim3(1), dim3(256), 0, stream, second, blocks2, blocks2, total, 1, (int)(sizeof(T) == 2),
                       found_inf, sum_squares, abs_max, 0u, 0u, owner, ticket);
    FS_HIP(hipGetLastError());
    return FSADAM_OK;
}

template <typename T>
int grad_plan_run(GradPlan* plan, float inv_scale, const float* inv_scale_dev, int write_back, float* found_inf, double* sum_squares,
                  float* abs_max, hipStream_t stream) {
    TableSlot& slot = plan->slots[plan->current];
    GradPartial* first = plan->d_partials;
    GradPartial* second = plan->d_partials + plan->cap_partials - kReduceBlocks - 1;
    GradPartial* total = second + kReduceBlocks;
    int rc = mark_order_after(slot.mark, stream);
    if (rc) return rc;
    rc = mark_order_after(plan->partials_mark, stream);
    if (rc) return rc;
    rc = grad_launch<T>(slot.d_table, plan->layout, plan->waves, plan->items, (size_t)plan->lds_throttle, inv_scale, inv_scale_dev, write_back,
                        first, second, total, found_inf, sum_squares, abs_max, stream);
    if (rc) return rc;
    rc = mark_use(slot.mark, stream, false);
    if (rc) return rc;
    return mark_use(plan->partials_mark, stream, false);
}

int validate_grads(const FsGradTensor* grads, int64_t n_tensors, int grad_dtype) {
    if (grad_dtype != FSADAM_GRAD_F32 && grad_dtype != FSADAM_GRAD_F16) return fail(FSADAM_EINVAL, "unknown gradient dtype " + std::to_string(grad_dtype));
    if (n_tensors < 1) return fail(FSADAM_EINVAL, "gradient list is empty");
    if (!grads) return fail(FSADAM_EINVAL, "grads is NULL");
    for (int64_t t = 0; t < n_tensors; ++t) {
        if (grads[t].numel < 0) return fail(FSADAM_EINVAL, "gradient " + std::to_string(t) + ": negative numel");
        if (grads[t].numel == 0) continue;
        if (!grads[t].g) return fail(FSADAM_EINVAL, "gradient " + std::to_string(t) + ": NULL pointer");
        if (!aligned_to(grads[t].g, grad_elem_size(grad_dtype))) return fail(FSADAM_EINVAL, "gradient " + std::to_string(t) + ": pointer not aligned to its element size");
    }
    return FSADAM_OK;
}

// ---- the variant of the gradient pass that allocates nothing ---------------------------------------

static_assert(sizeof(GradPartial) == 16 && sizeof(ChunkDesc) == 64 && kReduceBlocks == 512, "the scratch array is sized for these");
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;                  // guards the two arrays below; held for the whole of a call
unsigned char* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each GPU, once looked up
ChunkDesc g_scratch_staging[FSADAM_NOALLOC_MAX_DESCRIPTORS];  // host side of the table, rebuilt by every call

// Device address of this GPU's copy of `scratch` (every GPU that loads the library holds its own copy at
// its own address).  The symbol is resolved once per device, with that device current.
int scratch_on_current_device(unsigned char** out) {
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(FSADAM_EINVAL, "device index " + std::to_string(dev) + " is beyond what this entry point keeps a scratch pointer for");
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        FS_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        if (!ptr) return fail(FSADAM_EHIP, "hipGetSymbolAddress returned no address for the scratch array");
        g_scratch_ptr[dev] = static_cast<unsigned char*>(ptr);
    }
    *out = g_scratch_ptr[dev];
    return FSADAM_OK;
}

std::vector<GradPlan*> g_grad_cache;
constexpr size_t kGradCacheWays = 6;

bool same_grad_rows(const GradPlan* plan, const FsGradTensor* grads, int64_t n) {
    if ((int64_t)plan->rows.size() != n) return false;
    for (int64_t t = 0; t < n; ++t)
        if (plan->rows[t].g != grads[t].g || plan->rows[t].numel != grads[t].numel) return false;
    return true;
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

bool same_options(const Options& a, const Options& b) {
    return a.lds_throttle == b.lds_throttle && a.align_heads == b.align_heads && a.mid_tiles == b.mid_tiles && a.merge_runs == b.merge_runs &&
           a.upload_stream == b.upload_stream;
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
    if (k == "lds_throttle") {
        if (value < -1 || value > 65536) return fail(FSADAM_EINVAL, "lds_throttle must be -1 (per-mode default) or in [0, 65536] bytes");
        g_opt.lds_throttle = value;
    } else if (k == "align_heads") {
        if (value != 0 && value != 1) return fail(FSADAM_EINVAL, "align_heads must be 0 or 1");
        g_opt.align_heads = value;
    } else if (k == "merge_runs") {
        if (value != 0 && value != 1) return fail(FSADAM_EINVAL, "merge_runs must be 0 or 1");
        g_opt.merge_runs = value;
    } else if (k == "mid_tiles") {
        if (value < 0 || value > 64 || (value & (value - 1)) != 0) return fail(FSADAM_EINVAL, "mid_tiles must be 0 or a power of two up to 64");
        g_opt.mid_tiles = value;
    } else if (k == "upload_stream") {
        if (value != 0 && value != 1) return fail(FSADAM_EINVAL, "upload_stream must be 0 or 1");
        g_opt.upload_stream = value;
    } else if (k == "grad_items") {
        if (value != 0 && value != 2 && value != 4 && value != 8) return fail(FSADAM_EINVAL, "grad_items must be 0 (automatic), 2, 4 or 8");
        g_opt.grad_items = value;
    } else if (k == "grad_waves") {
        if (value != 0 && value != 1 && value != 4 && value != 16) return fail(FSADAM_EINVAL, "grad_waves must be 0 (automatic), 1, 4 or 16");
        g_opt.grad_waves = value;
    } else if (k == "grad_lds_throttle") {
        if (value < -1 || value > 65536) return fail(FSADAM_EINVAL, "grad_lds_throttle must be -1 (automatic) or in [0, 65536] bytes");
        g_opt.grad_lds_throttle = value;
    } else {
        return fail(FSADAM_EINVAL, "unknown option '" + k + "'");
    }
    return FSADAM_OK;
}

int fsadam_get_option(const char* name, int64_t* value) {
    if (!name || !value) return fail(FSADAM_EINVAL, "NULL argument");
    std::lock_guard<std::mutex> lock(g_mutex);
    const std::string k(name);
    if (k == "lds_throttle") *value = g_opt.lds_throttle;
    else if (k == "align_heads") *value = g_opt.align_heads;
    else if (k == "merge_runs") *value = g_opt.merge_runs;
    else if (k == "upload_stream") *value = g_opt.upload_stream;
    else if (k == "mid_tiles") *value = g_opt.mid_tiles;
    else if (k == "grad_items") *value = g_opt.grad_items;
    else if (k == "grad_lds_throttle") *value = g_opt.grad_lds_throttle;
    else if (k == "grad_waves") *value = g_opt.grad_waves;
    else return fail(FSADAM_EINVAL, "unknown option '" + k + "'");
    return FSADAM_OK;
}

int fsadam_layout(const FsAdamTensor* tensors, int64_t n_tensors, int precision_mode, FsAdamLayout* out, uint8_t* tensor_class,
                  uint8_t* vector_ok) {
    int rc = validate_rows(tensors, n_tensors, precision_mode);
    if (rc) return rc;
    if (!out) return fail(FSADAM_EINVAL, "out is NULL");
    Options opt;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        opt = g_opt;
    }
    std::vector<FsAdamTensor> runs;
    std::vector<int64_t> run_of;
    build_runs(tensors, n_tensors, precision_mode, opt.merge_runs != 0, runs, &run_of);
    std::vector<int64_t> heads;
    compute_heads(runs, precision_mode, opt, heads);
    const Layout L = compute_layout(runs, heads, precision_mode, opt);
    out->tile_elems = L.tile_elems;
    out->large_chunk_elems = L.large_chunk_elems;
    out->n_large_tensors = L.n_large;
    out->n_small_tensors = L.n_small;
    out->n_empty_tensors = 0;
    out->n_large_descriptors = L.n_large_descs;
    out->n_small_descriptors = L.n_small_descs;
    out->grid_large = L.large_blocks();
    out->grid_small = L.n_small_descs;
    out->mid_chunk_elems = L.mid_chunk_elems;
    out->n_mid_tensors = L.n_mid;
    out->n_mid_descriptors = L.n_mid_descs;
    out->grid_mid = L.mid_blocks();
    out->n_runs = L.n_runs;
    for (int64_t t = 0; t < n_tensors; ++t) {
        if (tensors[t].numel == 0) out->n_empty_tensors += 1;
        // a tensor is laid out with the run it belongs to
        const FsAdamTensor* run = run_of[(size_t)t] >= 0 ? &runs[(size_t)run_of[(size_t)t]] : nullptr;
        const int64_t head = run ? heads[(size_t)run_of[(size_t)t]] : 0;
        if (tensor_class) tensor_class[t] = run ? (uint8_t)class_of(run->numel - head, L) : 0;
        if (vector_ok) vector_ok[t] = (run && row_vector_ok(*run, precision_mode, head)) ? 1 : 0;
    }
    return FSADAM_OK;
}

int fsadam_head_elems(const FsAdamTensor* tensor, int precision_mode, int64_t* head) {
    if (!head) return fail(FSADAM_EINVAL, "head is NULL");
    int rc = validate_rows(tensor, 1, precision_mode);
    if (rc) return rc;
    Options opt;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        opt = g_opt;
    }
    *head = tensor->numel > 0 ? head_elems(*tensor, precision_mode, opt) : 0;
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

int fsadam_plan_lazy_events(FsAdamPlan* plan, int on) {
    if (!plan) return fail(FSADAM_EINVAL, "plan is NULL");
    if (on != 0 && on != 1) return fail(FSADAM_EINVAL, "lazy_events must be 0 or 1");
    if (!on) {  // from now on every use is followed by its event: catch up on the ones that are owed
        for (TableSlot& slot : plan->slots)
            if (int rc = mark_settle(slot.mark)) return rc;
    }
    plan->lazy_events = on != 0;
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
    return plan_step(plan, lr, beta1, beta2, eps, grad_scale, nullptr, optim_scale, decay, step, eps_mode, bias_correction,
                     found_inf_dev, static_cast<hipStream_t>(hip_stream));
}

int fsadam_plan_zero_state(FsAdamPlan* plan, void* hip_stream) {
    if (!plan) return fail(FSADAM_EINVAL, "plan is NULL");
    return plan_zero_state(plan, static_cast<hipStream_t>(hip_stream));
}

int fsadam_plan_step_dev_scale(FsAdamPlan* plan, float lr, float beta1, float beta2, float eps, const float* grad_scale_dev,
                               float optim_scale, float decay, int step, int eps_mode, int bias_correction,
                               float* found_inf_dev, void* hip_stream) {
    if (!plan) return fail(FSADAM_EINVAL, "plan is NULL");
    if (!grad_scale_dev) return fail(FSADAM_EINVAL, "grad_scale_dev is NULL");
    if (!aligned_to(grad_scale_dev, 4)) return fail(FSADAM_EINVAL, "grad_scale_dev is not aligned to 4 bytes");
    return plan_step(plan, lr, beta1, beta2, eps, 1.0f, grad_scale_dev, optim_scale, decay, step, eps_mode, bias_correction,
                     found_inf_dev, static_cast<hipStream_t>(hip_stream));
}

int fsadam_plan_info(const FsAdamPlan* plan, FsAdamPlanInfo* out) {
    if (!plan || !out) return fail(FSADAM_EINVAL, "NULL argument");
    std::memset(out, 0, sizeof(*out));
    const Layout& L = plan->layout;
    out->mode = plan->mode;
    out->device = plan->device;
    out->n_tensors = (int64_t)plan->rows.size();
    out->total_elems = L.total_elems;
    out->tile_elems = L.tile_elems;
    out->large_chunk_elems = L.large_chunk_elems;
    out->n_descriptors = L.descs();
    out->n_vector_tensors = L.n_vector;
    out->n_scalar_tensors = L.n_scalar;
    out->n_launches = L.descs() > 0 ? 1 : 0;
    out->grid = L.blocks();
    out->block = kBlock;
    out->n_runs = L.n_runs;
    out->lds_throttle = plan->lds_bytes;
    out->uploads = plan->uploads;
    return FSADAM_OK;
}

int fsadam_plan_destroy(FsAdamPlan* plan) {
    if (!plan) return FSADAM_OK;
    plan_release_buffers(plan);
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
    Options now;
    {
        std::lock_guard<std::mutex> lock(g_mutex);
        now = g_opt;
    }
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    FsAdamPlan* hit = nullptr;
    FsAdamPlan* victim = nullptr;
    for (FsAdamPlan* c : g_cache) {
        if (c->device == dev && c->mode == precision_mode && same_options(c->opt, now) && same_rows(c, tensors, n_tensors)) { hit = c; break; }
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
    return plan_step(hit, lr, beta1, beta2, eps, grad_scale, nullptr, optim_scale, decay, step, eps_mode, bias_correction,
                     found_inf_dev, stream);
}


int fsadam_grad_pass(const FsGradTensor* grads, int64_t n_tensors, int grad_dtype, float inv_scale, const float* inv_scale_dev,
                     int write_back, float* found_inf_dev, double* sum_squares_dev, float* abs_max_dev, void* hip_stream) {
    if (int bad = validate_grads(grads, n_tensors, grad_dtype)) return bad;
    int dev = -1;
    FS_HIP(hipGetDevice(&dev));
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    if (int refused = refuse_capture(stream)) return refused;  // its partial sums are guarded by events the host waits on
    int64_t cur_items, cur_lds, cur_waves, cur_heads, cur_mid, cur_upload;
    grad_shape(write_back != 0 && !(inv_scale_dev == nullptr && inv_scale == 1.0f), &cur_items, &cur_lds, &cur_waves, &cur_heads, &cur_mid, &cur_upload);
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    GradPlan* hit = nullptr;
    GradPlan* victim = nullptr;
    for (GradPlan* c : g_grad_cache) {
        if (c->device == dev && c->dtype == grad_dtype && c->items == cur_items && c->lds_throttle == cur_lds &&
            c->waves == cur_waves && c->align_heads == cur_heads && c->mid_tiles == cur_mid && same_grad_rows(c, grads, n_tensors)) { hit = c; break; }
        if (c->device == dev && c->dtype == grad_dtype && (!victim || c->lru < victim->lru)) victim = c;
    }
    if (!hit) {
        if (g_grad_cache.size() < kGradCacheWays || !victim) {
            GradPlan* fresh = new (std::nothrow) GradPlan();
            if (!fresh) return fail(FSADAM_ENOMEM, "out of host memory");
            fresh->device = dev;
            fresh->dtype = grad_dtype;
            fresh->items = cur_items;
            fresh->lds_throttle = cur_lds;
            if (g_grad_cache.size() >= kGradCacheWays) {
                size_t oldest = 0;
                for (size_t i = 1; i < g_grad_cache.size(); ++i) if (g_grad_cache[i]->lru < g_grad_cache[oldest]->lru) oldest = i;
                grad_plan_free(g_grad_cache[oldest]);
                g_grad_cache[oldest] = fresh;
            } else {
                g_grad_cache.push_back(fresh);
            }
            victim = fresh;
        }
        victim->items = cur_items;
        victim->lds_throttle = cur_lds;
        victim->align_heads = cur_heads;
        victim->mid_tiles = cur_mid;
        victim->own_upload_stream = cur_upload != 0;
        victim->waves = cur_waves;
        int rc = grad_plan_set(victim, grads, n_tensors, stream);
        if (rc) { victim->rows.clear(); return rc; }
        hit = victim;
    }
    hit->lru = ++g_tick;
    return grad_dtype == FSADAM_GRAD_F16
               ? grad_plan_run<_Float16>(hit, inv_scale, inv_scale_dev, write_back, found_inf_dev, sum_squares_dev, abs_max_dev, stream)
               : grad_plan_run<float>(hit, inv_scale, inv_scale_dev, write_back, found_inf_dev, sum_squares_dev, abs_max_dev, stream);
}

int fsadam_grad_pass_noalloc(const FsGradTensor* grads, int64_t n_tensors, int grad_dtype, float inv_scale, const float* inv_scale_dev,
                             int write_back, float* found_inf_dev, double* sum_squares_dev, float* abs_max_dev, void* hip_stream) {
    if (int bad = validate_grads(grads, n_tensors, grad_dtype)) return bad;
    hipStream_t stream = static_cast<hipStream_t>(hip_stream);
    // Shape: 16 tiles per workgroup whatever the kind of pass (one partial per workgroup keeps the scratch small);
    // vectors per lane and ballast as fsadam_grad_pass chooses them.  Options are not consulted.
    const bool writes = write_back != 0 && !(inv_scale_dev == nullptr && inv_scale == 1.0f);
    const int64_t waves = 16, items = writes ? 4 : 8;
    const size_t lds = writes ? 12288 : 16384;
    const Layout L = grad_layout(grads, n_tensors, grad_dtype, items, /*align_heads=*/1, /*mid_tiles=*/16);
    const int64_t n_descs = L.descs(), n_groups = ceil_div(L.blocks(), waves);
    if (n_descs > FSADAM_NOALLOC_MAX_DESCRIPTORS)
        return fail(FSADAM_EINVAL, "gradient list needs " + std::to_string(n_descs) + " descriptors, fsadam_grad_pass_noalloc holds at most " +
                                       std::to_string(FSADAM_NOALLOC_MAX_DESCRIPTORS) + " (use fsadam_grad_pass)");
    if (n_groups > FSADAM_NOALLOC_MAX_WORKGROUPS)
        return fail(FSADAM_EINVAL, "gradient list needs " + std::to_string(n_groups) + " workgroups, fsadam_grad_pass_noalloc holds partial results for at most " +
                                       std::to_string(FSADAM_NOALLOC_MAX_WORKGROUPS) + " (use fsadam_grad_pass)");
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    // every GPU has its own copy of the array: the one this call uses must be the one the stream runs on
    if (stream) {
        hipDevice_t stream_device = -1;
        int current = -1;
        FS_HIP(hipGetDevice(&current));
        if (hipStreamGetDevice(stream, &stream_device) != hipSuccess) {
            (void)hipGetLastError();
            return fail(FSADAM_EINVAL, "the stream could not be asked for its device");
        }
        if ((int)stream_device != current)
            return fail(FSADAM_EINVAL, "the stream belongs to device " + std::to_string((int)stream_device) + ", the current device is " + std::to_string(current));
    }
    unsigned char* base = nullptr;
    if (int rc = scratch_on_current_device(&base)) return rc;
    ChunkDesc* table = reinterpret_cast<ChunkDesc*>(base);
    GradPartial* first = reinterpret_cast<GradPartial*>(base + kScratchTableBytes);
    GradPartial* second = first + FSADAM_NOALLOC_MAX_WORKGROUPS + kSlotSlack;
    GradPartial* total = second + kReduceBlocks;
    if (!grad_fill_table(g_scratch_staging, L, grads, n_tensors, grad_elem_size(grad_dtype), 1))
        return fail(FSADAM_EINVAL, "internal error: descriptor count differs from the layout");
    // The table travels in kernel arguments, kDescsPerPut rows per launch: no copy engine, no staging buffer of
    // the runtime's, nothing a capture could not record.  The first of these launches (there is always one) takes
    // possession of the array for this call, the last reduction gives it back: see fsadam_put_descs.
    uint32_t* owner = reinterpret_cast<uint32_t*>(total + 1);
    static uint32_t next_ticket = 0;  // guarded by g_scratch_mutex
    if (++next_ticket == 0) ++next_ticket;
    const uint32_t ticket = next_ticket;
    int64_t at = 0;
    do {
        const int64_t count = std::min<int64_t>(kDescsPerPut, n_descs - at);
        DescBatch batch;
        std::memcpy(batch.rows, g_scratch_staging + at, (size_t)count * sizeof(ChunkDesc));
        hipLaunchKernelGGL(fsadam_put_descs, dim3(1), dim3(64), 0, stream, table, batch, (uint32_t)at, (uint32_t)count, owner, ticket);
        at += kDescsPerPut;
    } while (at < n_descs);
    FS_HIP(hipGetLastError());
    // Every partial a reduction reads was written by this call's tiles; nothing in the scratch has to start at zero
    // except the two words that say who owns it, which every call leaves at zero.
    return grad_dtype == FSADAM_GRAD_F16
               ? grad_launch<_Float16>(table, L, waves, items, lds, inv_scale, inv_scale_dev, write_back, first, second, total, found_inf_dev,
                                       sum_squares_dev, abs_max_dev, stream, owner, ticket)
               : grad_launch<float>(table, L, waves, items, lds, inv_scale, inv_scale_dev, write_back, first, second, total, found_inf_dev,
                                    sum_squares_dev, abs_max_dev, stream, owner, ticket);
}

int fsadam_clear_cache(void) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (FsAdamPlan* c : g_cache) fsadam_plan_destroy(c);
    g_cache.clear();
    for (GradPlan* c : g_grad_cache) grad_plan_free(c);
    g_grad_cache.clear();
    return FSADAM_OK;
}

}  // extern "C"
