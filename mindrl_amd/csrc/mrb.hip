// libmrb.so — C ABI (include/mrb.h) over the HIP kernels in mrb_kernels.h.
// Host side: handle registry, ring/tree bookkeeping, argument checks, launches.
// Nothing in this file computes a result on the CPU; without a HIP device every
// entry point that touches a buffer fails with MRB_EHIP.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cfloat>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "mrb_kernels.h"

namespace {

using namespace mrb;

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

#define HIP_TRY(expr)                                                                          \
    do {                                                                                       \
        hipError_t e_ = (expr);                                                                \
        if (e_ != hipSuccess) return fail(MRB_EHIP, "%s: %s", #expr, hipGetErrorString(e_));    \
    } while (0)

#define LAUNCH_CHECK(name)                                                                     \
    do {                                                                                       \
        hipError_t e_ = hipGetLastError();                                                     \
        if (e_ != hipSuccess) return fail(MRB_EHIP, "launch %s: %s", name, hipGetErrorString(e_)); \
    } while (0)

// Row storage. By default a structure of arrays, field i = [capacity, bytes_i] (reference layout:
// mindspore_rl/core/uniform_replay_buffer.py:26-47). With the library option "packed_rows" narrow rows are kept
// packed instead: one [capacity, row_stride] allocation, field i at byte offset_i of every row (each field
// aligned to its own copy granule), so that a sampled row's fields share cache lines instead of costing one
// 128-byte line per field. Either way row r of field i starts at data[i] + r * stride[i].
struct RowStore {
    int64_t capacity = 0;
    int nfields = 0;
    int64_t bytes[MRB_MAX_FIELDS] = {};
    int64_t stride[MRB_MAX_FIELDS] = {};
    uint8_t* data[MRB_MAX_FIELDS] = {};
    uint8_t* packed_base = nullptr;  // packed rows: the one allocation (data[i] point into it)
    uint32_t vec_log2[MRB_MAX_FIELDS] = {};
    uint32_t units[MRB_MAX_FIELDS] = {};
    int64_t row_split = 0;  // option "row_split": least number of workgroups per row in the wide-row kernel (0 = auto)
    int64_t row_wave = 0;   // option "row_wave": the wave-per-row sample kernel, 0 = for launches of many rows, 1 = whenever
                            // the rows fit it, 2 = never

    ~RowStore() {
        if (packed_base) {
            (void)hipFree(packed_base);
            return;
        }
        for (int i = 0; i < nfields; ++i)
            if (data[i]) (void)hipFree(data[i]);
    }
};

// Library-wide default of the option "packed_rows" (mrb_set_option with handle 0): buffers created afterwards
// keep their rows packed when a packed row takes at most this many bytes; 0 = every field an array of its own.
std::atomic<int64_t> g_packed_rows{0};

int rows_alloc(RowStore& r, int64_t capacity, int nfields, const int64_t* field_bytes) {
    if (capacity <= 0 || capacity > (1ll << 30)) return fail(MRB_EINVAL, "capacity %lld outside [1, 2^30]", (long long)capacity);
    if (nfields <= 0 || nfields > MRB_MAX_FIELDS) return fail(MRB_EINVAL, "nfields %d outside [1, %d]", nfields, MRB_MAX_FIELDS);
    if (!field_bytes) return fail(MRB_EINVAL, "field_bytes is NULL");
    for (int i = 0; i < nfields; ++i)
        if (field_bytes[i] <= 0 || field_bytes[i] > (1ll << 30))
            return fail(MRB_EINVAL, "field_bytes[%d] = %lld outside [1, 2^30]", i, (long long)field_bytes[i]);
    r.capacity = capacity;
    int64_t offset[MRB_MAX_FIELDS], end = 0, widest = 1;
    for (int i = 0; i < nfields; ++i) {
        r.bytes[i] = field_bytes[i];
        uint32_t vl = 4;
        while (vl > 0 && (field_bytes[i] & ((1ll << vl) - 1))) --vl;
        r.vec_log2[i] = vl;
        r.units[i] = (uint32_t)(field_bytes[i] >> vl);
        // where the field would lie in a packed row: at the next multiple of its own copy granule
        const int64_t g = 1ll << vl;
        offset[i] = (end + g - 1) / g * g;
        end = offset[i] + field_bytes[i];
        if (g > widest) widest = g;
    }
    const int64_t packed_row = (end + widest - 1) / widest * widest;  // rows start at multiples of the widest granule
    if (nfields > 1 && packed_row <= g_packed_rows.load()) {
        const size_t total = (size_t)capacity * (size_t)packed_row;
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&r.packed_base), total));
        HIP_TRY(hipMemset(r.packed_base, 0, total));
        for (int i = 0; i < nfields; ++i) {
            r.data[i] = r.packed_base + offset[i];
            r.stride[i] = packed_row;
        }
        r.nfields = nfields;
        return MRB_OK;
    }
    for (int i = 0; i < nfields; ++i) {
        const size_t total = (size_t)capacity * (size_t)field_bytes[i];
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&r.data[i]), total));
        r.nfields = i + 1;  // so the destructor frees what exists
        r.stride[i] = field_bytes[i];
        HIP_TRY(hipMemset(r.data[i], 0, total));
    }
    return MRB_OK;
}

// Builds the per-call field table. `io` pointers must honour each field's copy granule.
int make_table(const RowStore& r, const void* const* io, int64_t n, IoTable& t) {
    if (!io) return fail(MRB_EINVAL, "field pointer array is NULL");
    t.nfields = r.nfields;
    t.prefix[0] = 0;
    for (int i = 0; i < r.nfields; ++i) {
        if (!io[i]) return fail(MRB_EINVAL, "field %d pointer is NULL", i);
        if (reinterpret_cast<uintptr_t>(io[i]) & ((1u << r.vec_log2[i]) - 1))
            return fail(MRB_EINVAL, "field %d pointer %p is not %u-byte aligned", i, io[i], 1u << r.vec_log2[i]);
        t.store[i] = r.data[i];
        t.io[i] = const_cast<uint8_t*>(static_cast<const uint8_t*>(io[i]));
        t.row_bytes[i] = (uint32_t)r.bytes[i];
        t.stride[i] = (uint32_t)r.stride[i];
        t.units[i] = r.units[i];
        t.vec_log2[i] = r.vec_log2[i];
        t.prefix[i + 1] = t.prefix[i] + (uint64_t)n * r.units[i];
    }
    return MRB_OK;
}

uint32_t grid_for(uint64_t work, uint32_t per_thread = 1) {
    uint64_t g = (work + (uint64_t)kWG * per_thread - 1) / ((uint64_t)kWG * per_thread);
    if (g < 1) g = 1;
    if (g > 16384) g = 16384;
    return (uint32_t)g;
}

// One thread per entry, no grid-stride loop (n < 2^32, so the grid fits).
uint32_t grid_exact(uint64_t n) { return (uint32_t)((n + kWG - 1) / kWG); }

// Describes the append of rows [skip, skip + n) of the caller's matrices at ring position first_slot.
int put_args(const RowStore& r, const void* const* src, int64_t skip, int64_t n, int64_t first_slot, PutArgs& p) {
    const void* shifted[MRB_MAX_FIELDS];
    if (!src) return fail(MRB_EINVAL, "field pointer array is NULL");
    for (int i = 0; i < r.nfields; ++i) {
        if (!src[i]) return fail(MRB_EINVAL, "field %d pointer is NULL", i);
        shifted[i] = static_cast<const uint8_t*>(src[i]) + skip * r.bytes[i];
    }
    int rc = make_table(r, shifted, n, p.t);
    if (rc) return rc;
    p.capacity = r.capacity;
    p.first_slot = first_slot;
    p.src_capacity = 0;
    p.src_first = 0;
    p.blocks = grid_for(p.t.prefix[p.t.nfields]);
    return MRB_OK;
}

int rows_put(const RowStore& r, const void* const* src, int64_t skip, int64_t n, int64_t first_slot, hipStream_t s) {
    PutArgs p{};
    int rc = put_args(r, src, skip, n, first_slot, p);
    if (rc) return rc;
    hipLaunchKernelGGL(k_rows_put, dim3(p.blocks), dim3(kWG), 0, s, p);
    LAUNCH_CHECK("k_rows_put");
    return MRB_OK;
}

int64_t widest_field(const RowStore& r) {
    int64_t m = 0;
    for (int i = 0; i < r.nfields; ++i)
        if (r.bytes[i] > m) m = r.bytes[i];
    return m;
}

// Describes n rows of `r` for the wide-row kernels: one workgroup per row unless a row holds more than
// kMaxInFlight * kCopyThreads (2048) wide granules, or the buffer's "row_split" option asks for more.
// Returns the number of granules a copy thread holds (2 or 8) or 0 on error.
int wide_plan(const RowStore& r, const IoTable& t, int64_t n, WidePlan& plan, dim3& grid) {
    const uint32_t nbatch = plan.nbatch;
    plan = WidePlan{};
    plan.nbatch = nbatch;
    for (int i = 0; i < r.nfields; ++i) plan.nwide += r.vec_log2[i] == 4;
    plan.nnarrow = r.nfields - plan.nwide;
    int w = 0, m = plan.nwide;
    for (int i = 0; i < r.nfields; ++i) {
        const bool wide = r.vec_log2[i] == 4;
        const int q = wide ? w++ : m++;
        plan.f[q].src = t.store[i];
        plan.f[q].dst = t.io[i];
        plan.f[q].rb = t.row_bytes[i];
        plan.f[q].ss = t.stride[i];
        uint32_t& items = wide ? plan.wide_items : plan.narrow_items;
        plan.f[q].first = items;
        items += wide ? r.units[i] : t.row_bytes[i];
    }
    const uint32_t per_wg = (uint32_t)kMaxInFlight * kCopyThreads;
    uint32_t split = (plan.wide_items + per_wg - 1) / per_wg;
    if (r.row_split > (int64_t)split) split = (uint32_t)r.row_split;
    if (split < 1) split = 1;
    plan.split = (int)split;
    plan.share = (plan.wide_items + split - 1) / split;
    if (n > 0x7fffffffll || split > 65535u) {
        fail(MRB_EINVAL, "%lld rows of %u workgroups each exceed one launch", (long long)n, split);
        return 0;
    }
    grid = dim3((uint32_t)n, split);
    const uint32_t per_thread = (plan.share + kCopyThreads - 1) / kCopyThreads;  // <= kMaxInFlight
    return per_thread <= 2 ? 2 : 8;
}

// The descent plan of a tree of `depth` levels as the wide-row sample kernel takes it: bits 0-3 the
// number of node groups (one dependent load each), then 5 bits per group with its levels (<= 10).
uint32_t pack_groups(int depth) {
    const int count = (depth + kGroupMaxLevels - 1) / kGroupMaxLevels;
    uint32_t packed = (uint32_t)count;
    for (int i = 0; i < count; ++i) packed |= (uint32_t)(depth / count + (i < depth % count ? 1 : 0)) << (4 + 5 * i);
    return packed;
}
// The same with what else the sample kernels' `groups` word carries: bit 19 tells that the generator's call counter
// is on the device (the walk then reads it there; the flag is among the preloaded arguments, the counter's address
// is not), bits 20-31 the number of batches in the launch minus one.
uint32_t groups_word(const SampleArgs& a, int64_t nbatch) {
    return pack_groups(a.depth) | ((uint32_t)(nbatch - 1) << 20) | ((!a.uniforms && a.size < 0) ? 1u << 19 : 0u);
}

// Threads of a wide-row workgroup: the walker wave, the copy waves and, where rows have narrow fields, their wave.
inline uint32_t wide_threads(const WidePlan& plan) { return plan.narrow_items ? (uint32_t)kWideWG : (uint32_t)kWideWG - 64u; }

template <int kInF, bool kTen, bool kOneWide>
void launch_sample_wide(dim3 grid, const SampleArgs& a, const WidePlan& plan, hipStream_t s) {
    const SampleTail tail{a.mn, a.out_idx, a.out_w, a.err, a.size, a.beta};
    hipLaunchKernelGGL((k_per_sample_wide<kInF, kTen, kOneWide>), grid, dim3(wide_threads(plan)), 0, s, a.sum, a.uniforms, a.depth,
                       groups_word(a, plan.nbatch), (int)a.batch, (uint32_t)a.capacity, a.seed, a.calls, tail, plan);
}

template <int kInF>
void launch_sample_wide_as(dim3 grid, const SampleArgs& a, const WidePlan& plan, hipStream_t s) {
    const bool ten = a.depth > 0 && a.depth % kGroupMaxLevels == 0;  // every node group takes 10 levels
    const bool one = plan.nwide == 1;
    if (ten) one ? launch_sample_wide<kInF, true, true>(grid, a, plan, s) : launch_sample_wide<kInF, true, false>(grid, a, plan, s);
    else one ? launch_sample_wide<kInF, false, true>(grid, a, plan, s) : launch_sample_wide<kInF, false, false>(grid, a, plan, s);
}

// A sample call's optional second layer: field `row_field` of the row whose slot number the sampled row holds
// in its 8-byte field `slot_field` goes to `out` ([batch, row bytes]).
struct NextRows {
    int slot_field = -1, row_field = -1;
    void* out = nullptr;
};

constexpr int64_t kRowWaveMinRows = 2048;  // fewest rows of a launch that go to the wave-per-row sample kernel

template <int kInF, bool kTen, bool kOneWide>
void launch_sample_next(dim3 grid, const SampleArgs& a, const WidePlan& plan, const NextPlan& nx, hipStream_t s) {
    const SampleTail tail{a.mn, a.out_idx, a.out_w, a.err, a.size, a.beta};
    hipLaunchKernelGGL((k_per_sample_next<kInF, kTen, kOneWide>), grid, dim3(wide_threads(plan)), 0, s, a.sum, a.uniforms, a.depth,
                       groups_word(a, 1), (int)a.batch, (uint32_t)a.capacity, a.seed, a.calls, tail, plan, nx);
}

template <int kInF>
void launch_sample_next_as(dim3 grid, const SampleArgs& a, const WidePlan& plan, const NextPlan& nx, hipStream_t s) {
    const bool ten = a.depth > 0 && a.depth % kGroupMaxLevels == 0;
    const bool one = plan.nwide == 1;
    if (ten) one ? launch_sample_next<kInF, true, true>(grid, a, plan, nx, s) : launch_sample_next<kInF, true, false>(grid, a, plan, nx, s);
    else one ? launch_sample_next<kInF, false, true>(grid, a, plan, nx, s) : launch_sample_next<kInF, false, false>(grid, a, plan, nx, s);
}

int sample_wide(const RowStore& r, const SampleArgs& a, const IoTable& t, int64_t nbatch, hipStream_t s,
                const NextRows* next = nullptr) {
    WidePlan plan;
    dim3 grid;
    plan.nbatch = (uint32_t)nbatch;
    const int inflight = wide_plan(r, t, nbatch * a.batch, plan, grid);
    if (inflight == 0) return MRB_EINVAL;
    if (next) {
        // the second layer of workgroups: one wide field, split like a row of its own
        NextPlan nx{};
        const int f = next->row_field;
        nx.slot_field = r.data[next->slot_field];
        nx.plan.nwide = 1;
        nx.plan.nbatch = 1;
        nx.plan.f[0].src = r.data[f];
        nx.plan.f[0].dst = static_cast<uint8_t*>(next->out);
        nx.plan.f[0].rb = (uint32_t)r.bytes[f];
        nx.plan.f[0].ss = (uint32_t)r.stride[f];
        nx.slot_stride = (uint32_t)r.stride[next->slot_field];
        nx.plan.wide_items = r.units[f];
        const uint32_t per_wg = (uint32_t)kMaxInFlight * kCopyThreads;
        const uint32_t split = (nx.plan.wide_items + per_wg - 1) / per_wg;
        nx.plan.split = (int)split;
        nx.plan.share = (nx.plan.wide_items + split - 1) / split;
        if (split > 65535u) return fail(MRB_EINVAL, "field %d is too wide for one launch", f);
        if (split > grid.y) grid.y = split;
        grid.z = 2;
        const uint32_t per_thread = (nx.plan.share + kCopyThreads - 1) / kCopyThreads;
        if (inflight == 2 && per_thread <= 2) launch_sample_next_as<2>(grid, a, plan, nx, s);
        else launch_sample_next_as<8>(grid, a, plan, nx, s);
        LAUNCH_CHECK("k_per_sample_next");
        return MRB_OK;
    }
    // Many rows of up to 4 KB in 16-byte fields and a handful of narrow bytes: a wave per row (k_per_sample_rows)
    // instead of a workgroup per row. One wave does in a row what six do side by side, so a launch of few rows
    // takes longer that way (config 4, 1024 rows of 521 B: 6.4 us against 5.5) and a launch of many less (4096
    // rows: 9.2 us against 15.6; 16,384: 26 against 54): a sixth of the waves to dispatch. (`row_split` asks for
    // the workgroup kernel.)
    const int64_t nrows = nbatch * a.batch;
    if (r.row_split == 0 && r.row_wave != 2 && plan.split == 1 && plan.wide_items <= (uint32_t)kRowWaveInF * 64u &&
        plan.narrow_items <= 256u && (nrows >= kRowWaveMinRows || r.row_wave == 1)) {
        const SampleTail tail{a.mn, a.out_idx, a.out_w, a.err, a.size, a.beta};
        const uint32_t blocks = (uint32_t)((nrows + kRowWaveWG / 64 - 1) / (kRowWaveWG / 64));
        const uint32_t packed = groups_word(a, plan.nbatch);
        if (a.depth > 0 && a.depth % kGroupMaxLevels == 0)
            hipLaunchKernelGGL((k_per_sample_rows<true>), dim3(blocks), dim3(kRowWaveWG), 0, s, a.sum, a.uniforms, a.depth, packed,
                               (int)a.batch, (uint32_t)a.capacity, a.seed, a.calls, nrows, tail, plan);
        else
            hipLaunchKernelGGL((k_per_sample_rows<false>), dim3(blocks), dim3(kRowWaveWG), 0, s, a.sum, a.uniforms, a.depth, packed,
                               (int)a.batch, (uint32_t)a.capacity, a.seed, a.calls, nrows, tail, plan);
        LAUNCH_CHECK("k_per_sample_rows");
        return MRB_OK;
    }
    // Fewer rows of that size: the workgroup kernel with two copy waves instead of four (k_per_sample_light).
    if (r.row_split == 0 && plan.split == 1 && plan.wide_items <= 2u * 64u * kLightCopyWaves && a.depth != 22) {
        const SampleTail tail{a.mn, a.out_idx, a.out_w, a.err, a.size, a.beta};
        const uint32_t packed = groups_word(a, plan.nbatch);
        const dim3 threads(plan.narrow_items ? (uint32_t)kLightWG : (uint32_t)kLightWG - 64u);
        const bool ten = a.depth > 0 && a.depth % kGroupMaxLevels == 0, one = plan.nwide == 1;
#define MRB_LAUNCH_LIGHT(T, O)                                                                                         \
    hipLaunchKernelGGL((k_per_sample_light<T, O>), grid, threads, 0, s, a.sum, a.uniforms, a.depth, packed, (int)a.batch, \
                       (uint32_t)a.capacity, a.seed, a.calls, tail, plan)
        if (ten) { if (one) MRB_LAUNCH_LIGHT(true, true); else MRB_LAUNCH_LIGHT(true, false); }
        else { if (one) MRB_LAUNCH_LIGHT(false, true); else MRB_LAUNCH_LIGHT(false, false); }
#undef MRB_LAUNCH_LIGHT
        LAUNCH_CHECK("k_per_sample_light");
        return MRB_OK;
    }
    if (inflight == 2) launch_sample_wide_as<2>(grid, a, plan, s);
    else launch_sample_wide_as<8>(grid, a, plan, s);
    LAUNCH_CHECK("k_per_sample_wide");
    return MRB_OK;
}

template <int kInF>
void launch_gather_wide(dim3 grid, const int64_t* indices, int mode, int64_t count, int64_t fixed_slot, uint64_t seed,
                        uint64_t calls, int64_t* out_indices, uint32_t* err, const WidePlan& plan, hipStream_t s) {
    if (plan.nwide == 1)
        hipLaunchKernelGGL((k_rows_gather_wide<kInF, true>), grid, dim3(wide_threads(plan)), 0, s, indices, mode, count, fixed_slot, seed,
                           calls, out_indices, err, plan);
    else
        hipLaunchKernelGGL((k_rows_gather_wide<kInF, false>), grid, dim3(wide_threads(plan)), 0, s, indices, mode, count, fixed_slot, seed,
                           calls, out_indices, err, plan);
}

// Gather of n rows whose slots are given (indices), drawn from the generator (indices NULL,
// fixed_slot < 0) or one fixed slot. Rows with a field of at least 1 KB go through the wide-row
// kernel (a workgroup per row, all loads before the first store), narrow rows through the flat kernel.
int gather_rows(const RowStore& r, const int64_t* indices, int64_t fixed_slot, int64_t count, uint64_t seed,
                uint64_t calls, int64_t n, int64_t* out_indices, void* const* dst_fields, uint32_t* err,
                hipStream_t s) {
    IoTable t;
    int rc = make_table(r, dst_fields, n, t);
    if (rc) return rc;
    if (widest_field(r) >= 1024 && n <= (1ll << 24)) {
        const int mode = fixed_slot >= 0 ? kFromFixedSlot : (indices ? kFromIndices : kFromGenerator);
        WidePlan plan;
        dim3 grid;
        plan.nbatch = 1;
        switch (wide_plan(r, t, n, plan, grid)) {
            case 0: return MRB_EINVAL;
            case 2: launch_gather_wide<2>(grid, indices, mode, count, fixed_slot, seed, calls, out_indices, err, plan, s); break;
            default: launch_gather_wide<8>(grid, indices, mode, count, fixed_slot, seed, calls, out_indices, err, plan, s); break;
        }
        LAUNCH_CHECK("k_rows_gather_wide");
        return MRB_OK;
    }
    // a row of workgroups per field, as many as the field with the most granules needs
    uint64_t most = 0;
    for (int f = 0; f < t.nfields; ++f) most = std::max<uint64_t>(most, t.prefix[f + 1] - t.prefix[f]);
    hipLaunchKernelGGL(k_rows_gather, dim3(grid_for(most), (uint32_t)t.nfields), dim3(kWG), 0, s, t, r.capacity, count,
                       indices, fixed_slot, seed, calls, out_indices, err);
    LAUNCH_CHECK("k_rows_gather");
    return MRB_OK;
}

// ---- the allocation-free entry point's scratch (mrb_per_update_noalloc) -------------------------
// Device memory that exists from the moment the library is loaded: callers that must not allocate
// (HIP graph capture, serving loops, harnesses that forbid hipMalloc) get the update_priorities
// scratch from here. Every device holds its own copy at its own address; `scratch` itself is only
// the host-side name of the symbol and is never passed to a kernel.
constexpr int64_t kNoAllocMaxEntries = 1 << 18;  // 1 MiB per device
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};

}  // namespace

static __device__ __align__(256) float scratch[1 << 18];

namespace {

// Address of the current device's copy of `scratch`, looked up once per device.
int static_scratch(float** out) {
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail(MRB_EINVAL, "device %d outside [0, %d)", dev, kMaxDevices);
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        float* p = nullptr;
        HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return MRB_OK;
}

struct Urb {
    RowStore rows;
    int64_t count = 0, head = 0;
    uint64_t seed = 0, calls = 0;
    uint32_t* err = nullptr;       // 16 bytes of flags, then the device copy of the counters (kUrb* in mrb_kernels.h)
    int64_t* counters = nullptr;   // = err + 16 bytes
    int64_t* slots = nullptr;      // device array of kUrbDrawMax slots: drawn there when the counters live on the device
    int64_t device_counters = 0;   // option "device_counters"
    ~Urb() {
        if (err) (void)hipFree(err);
        if (slots) (void)hipFree(slots);
    }
};

// count / head after appending n rows (write position chosen once per call: `count` while the
// buffer has never wrapped, else `head`).
void urb_advance(Urb& b, int64_t n) {
    const int64_t cap = b.rows.capacity;
    if (b.count < cap && b.head == 0) {
        const int64_t room = cap - b.count;
        if (n <= room) {
            b.count += n;
        } else {
            b.count = cap;
            b.head = (n - room) % cap;
        }
    } else {
        b.head = (b.head + n) % cap;
        b.count = b.count + n < cap ? b.count + n : cap;
    }
}

struct Per {
    RowStore rows;
    int64_t leaves = 1;
    int depth = 0;
    int64_t size = 0, pushes = 0;
    float alpha = 1.0f;
    float* sum = nullptr;
    float* mn = nullptr;
    unsigned long long* stamp = nullptr;
    float* maxp = nullptr;
    // sparse plan for very large trees (see k_tree_sparse): lowest s_g0 levels per entry, then s_rounds tile rounds
    int s_g0 = 0, s_rounds = 0, s_top = 0;
    int s_lo[kMaxRounds] = {}, s_g[kMaxRounds] = {};
    uint32_t* s_dirty[kMaxRounds] = {};
    // scratch of update_priorities (p^alpha of the call's entries): sized at create; a call with more
    // entries gets a larger array and the old one is kept until destroy (work may still be queued on it)
    float* powered = nullptr;
    int64_t powered_cap = 0;
    std::vector<float*> retired;
    uint32_t* err = nullptr;
    uint32_t* dirty[kMaxRounds] = {};
    int nrounds = 0;
    int lo[kMaxRounds] = {};
    int g[kMaxRounds] = {};
    int top_depth = 0;
    uint64_t epoch = 0;
    uint64_t seed = 0, calls = 0;
    int device = 0;           // the HIP device the buffer lives on
    int64_t sample_path = 0;  // option "sample_path": 0 = choose by row size, 1 = wide-row kernel, 2 = LDS-top kernel
    int64_t lds_levels = 0;   // option "lds_levels": tree levels staged in LDS by the LDS-top kernel (0 = auto)
    int64_t fused = 1;        // option "fused_rebuild": small updates and pushes rebuild the tree in one launch
    int64_t* counters = nullptr;   // device copy of pushes / size / calls (Counters in mrb_kernels.h)
    int64_t device_counters = 0;   // option "device_counters": kernels read the counters from the device
    ~Per() {
        if (sum) (void)hipFree(sum);
        if (mn) (void)hipFree(mn);
        if (stamp) (void)hipFree(stamp);
        if (powered) (void)hipFree(powered);
        for (auto* d : retired) (void)hipFree(d);
        for (auto* d : s_dirty)
            if (d) (void)hipFree(d);
        if (err) (void)hipFree(err);
        for (auto* d : dirty)
            if (d) (void)hipFree(d);
    }
};

struct Res {
    RowStore rows;
    int64_t size = 0, total = 0;
    uint64_t seed = 0, calls = 0, epoch = 0;
    unsigned long long* stamp = nullptr;
    uint32_t* err = nullptr;
    ~Res() {
        if (stamp) (void)hipFree(stamp);
        if (err) (void)hipFree(err);
    }
};

std::mutex g_mu;
int64_t g_next = 1;
std::unordered_map<int64_t, std::shared_ptr<Urb>> g_urb;
std::unordered_map<int64_t, std::shared_ptr<Per>> g_per;
std::unordered_map<int64_t, std::shared_ptr<Res>> g_res;

std::shared_ptr<Urb> find_urb(int64_t h) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_urb.find(h);
    return it == g_urb.end() ? nullptr : it->second;
}
std::shared_ptr<Per> find_per(int64_t h) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_per.find(h);
    return it == g_per.end() ? nullptr : it->second;
}

std::shared_ptr<Res> find_res(int64_t h) {
    std::lock_guard<std::mutex> lk(g_mu);
    auto it = g_res.find(h);
    return it == g_res.end() ? nullptr : it->second;
}
#define GET_RES(b, h)                                                              \
    auto b = find_res(h);                                                          \
    if (!b) return fail(MRB_EHANDLE, "unknown reservoir buffer handle %lld", (long long)(h))
#define GET_URB(b, h)                                                              \
    auto b = find_urb(h);                                                          \
    if (!b) return fail(MRB_EHANDLE, "unknown uniform buffer handle %lld", (long long)(h))
#define GET_PER(b, h)                                                              \
    auto b = find_per(h);                                                          \
    if (!b) return fail(MRB_EHANDLE, "unknown priority buffer handle %lld", (long long)(h))

int read_and_clear_flags(uint32_t* d_err, uint32_t* flags, hipStream_t s) {
    uint32_t v = 0;
    HIP_TRY(hipMemcpyAsync(&v, d_err, sizeof(v), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    if (v) {
        HIP_TRY(hipMemsetAsync(d_err, 0, sizeof(v), s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    if (flags) *flags = v;
    return MRB_OK;
}

// Leaf tiles that n consecutive slots of the ring can meet wherever they start: ceil(n / 256) + 1 for the
// misalignment, one more where the slots wrap around the ring's end; never more than the ring's tiles.
uint32_t push_units(const UpdateArgs& a) {
    const uint64_t ring_tiles = ((uint64_t)a.capacity + kBlockNodes - 1) / kBlockNodes;
    const uint64_t units = ((uint64_t)a.n + kBlockNodes - 1) / kBlockNodes + 2;
    return (uint32_t)(units < ring_tiles ? units : ring_tiles);
}

// A push whose tree work is ONE launch and that also moves the device's counters on (a.advance != 0): every
// workgroup that rides along reports to one counter when it has read the ring position (see counters_push_done),
// which is worth it for a few dozen workgroups only - a larger copy then gets a launch of its own, ahead.
constexpr uint32_t kRideWithCounters = 64;
int ride_alone_if_large(const UpdateArgs& a, PutArgs& put, hipStream_t s) {
    if (a.advance && put.blocks > kRideWithCounters) {
        hipLaunchKernelGGL(k_rows_put, dim3(put.blocks), dim3(kWG), 0, s, put);
        LAUNCH_CHECK("k_rows_put");
        put.blocks = 0;
    }
    return MRB_OK;
}

// Rebuilds the tree above the leaves that `a` writes: one launch per round, then the top. A push hands
// its row copy over (`ride`): it is done by extra workgroups of the first launch.
int tree_rebuild(Per& b, UpdateArgs a, hipStream_t s, const PutArgs* ride = nullptr) {
    PutArgs none{};  // blocks == 0: no copy rides along
    // One round below the top and at most 16 waves of work (an update: a wave per entry; a push that does
    // not wrap: a wave per leaf tile under its slots): one launch of one workgroup that goes on to the top.
    // (More units per wave do not pay: the 16 waves of a workgroup share one compute unit's issue slots, and a
    // second unit costs a wave as much as the second launch it would save; four cost twice as much.)
    if (a.nrounds == 1 && b.fused) {
        uint32_t units = 0, tile_base = 0;
        if (a.inline_election) {
            units = (uint32_t)a.n;
        } else if (!a.indices && a.first_slot < 0) {
            units = push_units(a);  // the slots' start is only known on the device
        } else if (!a.indices && a.first_slot + a.n <= a.capacity) {
            tile_base = (uint32_t)(a.first_slot / kBlockNodes);
            units = (uint32_t)((a.first_slot + a.n - 1) / kBlockNodes) - tile_base + 1;
        }
        if (units > 0 && units <= (uint32_t)(kFusedWG / 64)) {
            PutArgs put = ride ? *ride : none;
            if (int rc = ride_alone_if_large(a, put, s)) return rc;
            put.blocks = (put.blocks + 3) / 4;  // the ride-along copy was sized for workgroups a quarter as large
            a.readers = 1 + put.blocks;         // (a.advance != 0: this one launch also moves the device's counters on)
            hipLaunchKernelGGL(k_tree_fused, dim3(1 + put.blocks), dim3(kFusedWG), 0, s, a, tile_base, units, put);
            LAUNCH_CHECK("k_tree_fused");
            return MRB_OK;
        }
    }
    // A push of at most 1024 rows into a tree of at most 16 levels is one launch: the single workgroup of
    // k_tree_top starts at the leaf level and skips the tiles outside the slot range (such a call is
    // launch-bound, not work-bound). Measured on 16,384 leaves: 6.3 us instead of 8.0. Updates keep their
    // leaf round: their waves scan the entries, which one workgroup does more slowly (11.5 vs 9.8 us).
    if (a.nrounds > 0 && !a.indices && a.n <= 1024 && a.depth <= 16) {
        a.nrounds = 0;
        a.top_depth = a.depth;
    }
    for (int r = 0; r < a.nrounds; ++r) {
        uint32_t tiles = (1u << a.lo[r]) / kBlockNodes;
        uint32_t tile_base = 0;
        if (r == 0 && !a.indices && a.first_slot < 0) {
            // a push whose first slot only the device knows: enough waves for every tile the slots can meet;
            // the kernel places them (tile_base carries their number)
            tiles = push_units(a);
            tile_base = tiles;
        } else if (r == 0 && !a.indices && a.first_slot + a.n <= a.capacity) {
            // a push that does not wrap: only the leaf tiles under its slot range need a wave
            tile_base = (uint32_t)(a.first_slot / kBlockNodes);
            tiles = (uint32_t)((a.first_slot + a.n - 1) / kBlockNodes) - tile_base + 1;
        }
        const PutArgs& put = (r == 0 && ride) ? *ride : none;
        if (r == 0 && a.inline_election) tiles = (a.n > kPairedAbove ? 2u : 1u) * (uint32_t)a.n;  // one or two waves per entry (see k_tree_update)
        hipLaunchKernelGGL(k_tree_update, dim3((tiles + 3) / 4 + put.blocks), dim3(kWG), 0, s, a.indices, a.priorities, a.sum, a.mn,
                           a.n, a.capacity, r | a.lo[r] << 8 | a.g[r] << 16, a.alpha, a, tile_base, put);
        LAUNCH_CHECK("k_tree_update");
    }
    PutArgs put = (a.nrounds == 0 && ride) ? *ride : none;
    if (int rc = ride_alone_if_large(a, put, s)) return rc;
    // the top is the call's last launch: it moves the device's counters on (a.advance != 0); only when it is also
    // the first do its workgroups read the ring position
    a.readers = a.nrounds == 0 ? 1 + put.blocks : 0;
    hipLaunchKernelGGL(k_tree_top, dim3(1 + put.blocks), dim3(kTopWG), 0, s, a, put);
    LAUNCH_CHECK("k_tree_top");
    return MRB_OK;
}

// Zero-fills `bytes` (a multiple of 4) of device memory with a kernel.
void fill_zero(void* p, size_t bytes, hipStream_t s) {
    const uint64_t n = bytes / sizeof(float);
    hipLaunchKernelGGL(k_fill_f32, dim3(grid_for(n)), dim3(kWG), 0, s, static_cast<float*>(p), 0.0f, n);
}

// Starts a new tree-update epoch. Epochs tag stamps and dirty words so that
// neither needs clearing between calls; when the 32-bit tag would wrap, both
// are cleared once.
int next_epoch(Per& b, hipStream_t s) {
    b.epoch += 1;
    if ((uint32_t)b.epoch == 0) {
        // cleared by a fill kernel, not a memset node: a caller may be capturing this stream (0.0f is all-zero bits)
        fill_zero(b.stamp, sizeof(unsigned long long) * (size_t)b.leaves, s);
        for (int r = 0; r < b.nrounds; ++r) fill_zero(b.dirty[r], sizeof(uint32_t) * ((size_t)1 << (b.lo[r] - b.g[r])), s);
        for (int r = 0; r < b.s_rounds; ++r)
            fill_zero(b.s_dirty[r], sizeof(uint32_t) * ((size_t)1 << (b.s_lo[r] - b.s_g[r])), s);
        LAUNCH_CHECK("k_fill_f32");
        b.epoch += 1;
    }
    return MRB_OK;
}

UpdateArgs update_args(Per& b) {
    UpdateArgs a{};
    a.capacity = b.rows.capacity;
    a.leaves = b.leaves;
    a.depth = b.depth;
    a.alpha = b.alpha;
    a.epoch = (uint32_t)b.epoch;
    a.stamp = b.stamp;
    a.sum = b.sum;
    a.mn = b.mn;
    a.maxp = b.maxp;
    a.maxp_next = b.maxp + 1;
    a.err = b.err;
    a.nrounds = b.nrounds;
    for (int r = 0; r < kMaxRounds; ++r) {
        a.dirty[r] = b.dirty[r];
        a.lo[r] = b.lo[r];
        a.g[r] = b.g[r];
    }
    a.top_depth = b.top_depth;
    return a;
}

// Most entries of an update that elect the last writer of each leaf among themselves (a wave per entry scans
// the call's entries); larger calls take the stamp pass (2048 measured: config 4's update 14.0 us against 14.7 with the pass, at twice the waves and four times the comparisons: not taken).
constexpr int64_t kElectMax = 1024;

// update_priorities on buffer b with `powered` (device f32[n]) as the scratch that holds the entries'
// p^alpha between the stamp pass and the leaf writes. Allocates nothing.
int per_update(Per& pb, const int64_t* indices, const float* priorities, int64_t n, float* powered, hipStream_t s) {
    Per* b = &pb;
    if (b->device_counters && n > kElectMax)
        return fail(MRB_ESTATE, "with device_counters an update takes at most 1024 entries (larger ones elect their "
                                "entries with tags the host counts, which a graph replay would repeat)");
    if (n > kElectMax) {
        // the stamp pass tags leaves with an epoch the HOST counts: a recording would freeze it, and replays would
        // elect entries against stale tags. Refused while the stream is being captured (a host-side query).
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        HIP_TRY(hipStreamIsCapturing(s, &st));
        if (st != hipStreamCaptureStatusNone)
            return fail(MRB_ESTATE, "an update of more than %lld entries cannot be recorded into a HIP graph (its "
                                    "election tags are counted on the host); split it into calls of at most %lld",
                        (long long)kElectMax, (long long)kElectMax);
    }
    int rc = next_epoch(*b, s);
    if (rc) return rc;
    UpdateArgs a = update_args(*b);
    a.powered = powered;
    a.indices = indices;
    a.priorities = priorities;
    a.n = n;
    // Few entries (but more than the 1024 that elect among themselves, below) on a very large tree: rebuild
    // the lowest levels per entry, not per tile.
    const bool sparse = b->s_g0 > 0 && n > kElectMax && n <= (b->leaves >> 8);
    if (sparse) {
        a.sparse_g0 = b->s_g0;
        a.nrounds = b->s_rounds;
        a.top_depth = b->s_top;
        for (int r = 0; r < kMaxRounds; ++r) {
            a.dirty[r] = b->s_dirty[r];
            a.lo[r] = b->s_lo[r];
            a.g[r] = b->s_g[r];
        }
    }
    // Up to a few hundred entries on a small tree: one workgroup, a thread per entry, walks the paths in one launch
    // (k_tree_wg; on deeper trees or with more entries one compute unit's memory traffic costs more than a launch.
    // On these trees it also beats the one-wave kernel below for 64 entries or fewer: 5.45 against 5.87 us at 64.)
    if (!sparse && b->fused && n <= kWgBestEntries && b->depth >= 2 && b->depth <= kWgMaxDepth) {
        // (65 to 128 entries: 1024 threads, eight per entry - the kernel's one-step path below the staged top)
        const uint32_t threads = n > 64 && n <= 128 ? 1024u : n <= kWgMinThreads ? (uint32_t)kWgMinThreads : (uint32_t)((n + 63) / 64 * 64);
        hipLaunchKernelGGL(k_tree_wg, dim3(1), dim3(threads), 0, s, a.indices, a.priorities, a.sum, a.mn, a.maxp, (int)a.n,
                           a.depth, (int)a.capacity, a.alpha, a);
        LAUNCH_CHECK("k_tree_wg");
        return MRB_OK;
    }
    // At most 64 entries on a deeper tree: one wave walks the entries' paths, leaves to root, in one launch (k_tree_paths).
    if (!sparse && b->fused && n <= kPathEntries && b->depth <= kPathMaxDepth) {
        hipLaunchKernelGGL(k_tree_paths, dim3(1), dim3(64), 0, s, a);
        LAUNCH_CHECK("k_tree_paths");
        return MRB_OK;
    }
    // A small call on a tree of at least four leaves needs no stamp pass: the leaf-level waves scan the
    // entries themselves (one launch less).
    if (!sparse && n <= kElectMax && b->depth >= 2) {
        a.inline_election = 1;
        return tree_rebuild(*b, a, s);
    }
    hipLaunchKernelGGL(k_update_stamp, dim3(grid_exact((uint64_t)n)), dim3(kWG), 0, s, a);
    LAUNCH_CHECK("k_update_stamp");
    if (!sparse) return tree_rebuild(*b, a, s);
    hipLaunchKernelGGL(k_tree_sparse, dim3(grid_exact((uint64_t)n << (b->s_g0 - 2))), dim3(kWG), 0, s, a);
    LAUNCH_CHECK("k_tree_sparse");
    const PutArgs none{};
    for (int r = 0; r < b->s_rounds; ++r) {
        const uint32_t tiles = (1u << b->s_lo[r]) / kBlockNodes;
        hipLaunchKernelGGL(k_tree_update, dim3((tiles + 3) / 4), dim3(kWG), 0, s, a.indices, a.priorities, a.sum, a.mn, a.n,
                           a.capacity, r | a.lo[r] << 8 | a.g[r] << 16, a.alpha, a, 0u, none);
        LAUNCH_CHECK("k_tree_update");
    }
    hipLaunchKernelGGL(k_tree_top, dim3(1), dim3(kTopWG), 0, s, a, none);
    LAUNCH_CHECK("k_tree_top");
    return MRB_OK;
}


// Device-resident counters: host -> device (when the option is switched on, after a load) and back (state
// queries, when it is switched off). Both wait for the device.
int counters_to_device(Per& b) {
    const int64_t v[kCntWords] = {b.pushes, b.size, (int64_t)b.calls, 0, b.pushes % b.rows.capacity};
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(b.counters, v, sizeof(v), hipMemcpyHostToDevice));
    return MRB_OK;
}
int counters_from_device(Per& b) {
    int64_t v[kCntWords];
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(v, b.counters, sizeof(v), hipMemcpyDeviceToHost));
    b.pushes = v[kCntPushes], b.size = v[kCntSize], b.calls = (uint64_t)v[kCntCalls];
    return MRB_OK;
}
int counters_to_device(Urb& b) {
    const int64_t cap = b.rows.capacity;
    const int64_t v[kCntWords] = {0, b.count, (int64_t)b.calls, b.head, b.count < cap && b.head == 0 ? b.count : b.head};
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(b.counters, v, sizeof(v), hipMemcpyHostToDevice));
    return MRB_OK;
}
int counters_from_device(Urb& b) {
    int64_t v[kCntWords];
    HIP_TRY(hipDeviceSynchronize());
    HIP_TRY(hipMemcpy(v, b.counters, sizeof(v), hipMemcpyDeviceToHost));
    b.count = v[kUrbCount], b.head = v[kUrbHead], b.calls = (uint64_t)v[kUrbCalls];
    return MRB_OK;
}
int counters_advance(Urb& b, int64_t rows, int64_t calls, hipStream_t s) {
    hipLaunchKernelGGL(k_urb_advance, dim3(1), dim3(64), 0, s, b.counters, rows, b.rows.capacity, calls);
    LAUNCH_CHECK("k_urb_advance");
    return MRB_OK;
}
int counters_advance(Per& b, int64_t pushed, int64_t calls, hipStream_t s) {
    hipLaunchKernelGGL(k_counters_advance, dim3(1), dim3(64), 0, s, b.counters, pushed, b.rows.capacity, calls);
    LAUNCH_CHECK("k_counters_advance");
    return MRB_OK;
}

}  // namespace

extern "C" {

const char* mrb_last_error(void) { return g_err; }
int mrb_backend(void) { return 1; }
int mrb_version(void) { return MRB_ABI_VERSION; }

int mrb_set_option(int64_t h, const char* name, int64_t value) {
    if (!name) return fail(MRB_EINVAL, "option name is NULL");
    if (h == 0) {
        // library-wide defaults, taken by buffers created afterwards
        if (strcmp(name, "packed_rows")) return fail(MRB_EINVAL, "'%s' is not a library-wide option (handle 0)", name);
        if (value < 0 || value > 4096) return fail(MRB_EINVAL, "packed_rows must be in [0, 4096] bytes");
        g_packed_rows.store(value);
        return MRB_OK;
    }
    RowStore* rows = nullptr;
    std::shared_ptr<Per> per = find_per(h);
    std::shared_ptr<Urb> urb = per ? nullptr : find_urb(h);
    std::shared_ptr<Res> res = (per || urb) ? nullptr : find_res(h);
    if (per) rows = &per->rows;
    if (urb) rows = &urb->rows;
    if (res) rows = &res->rows;
    if (!rows) return fail(MRB_EHANDLE, "unknown buffer handle %lld", (long long)h);
    if (!strcmp(name, "row_split")) {
        if (value < 0 || value > 64) return fail(MRB_EINVAL, "row_split must be in [0, 64]");
        rows->row_split = value;
    } else if (!strcmp(name, "row_wave")) {
        if (value < 0 || value > 2) return fail(MRB_EINVAL, "row_wave must be 0, 1 or 2");
        rows->row_wave = value;
    } else if (!strcmp(name, "sample_path")) {
        if (!per) return fail(MRB_EINVAL, "sample_path is an option of prioritized buffers");
        if (value < 0 || value > 2) return fail(MRB_EINVAL, "sample_path must be 0, 1 or 2");
        per->sample_path = value;
    } else if (!strcmp(name, "lds_levels")) {
        if (!per) return fail(MRB_EINVAL, "lds_levels is an option of prioritized buffers");
        if (value < 0 || value > 12) return fail(MRB_EINVAL, "lds_levels must be in [0, 12]");
        per->lds_levels = value;
    } else if (!strcmp(name, "device_counters")) {
        if (!per && !urb) return fail(MRB_EINVAL, "device_counters is an option of prioritized and uniform buffers");
        if (value < 0 || value > 1) return fail(MRB_EINVAL, "device_counters must be 0 or 1");
        if (per && value != per->device_counters) {
            const int rc = value ? counters_to_device(*per) : counters_from_device(*per);
            if (rc) return rc;
            per->device_counters = value;
        }
        if (urb && value != urb->device_counters) {
            const int rc = value ? counters_to_device(*urb) : counters_from_device(*urb);
            if (rc) return rc;
            urb->device_counters = value;
        }
    } else if (!strcmp(name, "fused_rebuild")) {
        if (!per) return fail(MRB_EINVAL, "fused_rebuild is an option of prioritized buffers");
        if (value < 0 || value > 1) return fail(MRB_EINVAL, "fused_rebuild must be 0 or 1");
        per->fused = value;
    } else {
        return fail(MRB_EINVAL, "unknown option '%s'", name);
    }
    return MRB_OK;
}

int mrb_field_layout(int64_t h, int field, void** dev_ptr, int64_t* row_stride) {
    const RowStore* rows = nullptr;
    std::shared_ptr<Per> per = find_per(h);
    std::shared_ptr<Urb> urb = per ? nullptr : find_urb(h);
    std::shared_ptr<Res> res = (per || urb) ? nullptr : find_res(h);
    if (per) rows = &per->rows;
    if (urb) rows = &urb->rows;
    if (res) rows = &res->rows;
    if (!rows) return fail(MRB_EHANDLE, "unknown buffer handle %lld", (long long)h);
    if (field < 0 || field >= rows->nfields) return fail(MRB_EINVAL, "bad field %d", field);
    if (dev_ptr) *dev_ptr = rows->data[field];
    if (row_stride) *row_stride = rows->stride[field];
    return MRB_OK;
}

/* ---------------------------------------------------------------- uniform */

int mrb_urb_create(int64_t capacity, int nfields, const int64_t* field_bytes, int64_t* out_handle) {
    if (!out_handle) return fail(MRB_EINVAL, "out_handle is NULL");
    if (capacity > 0x7fffffffll) return fail(MRB_EINVAL, "capacity %lld does not fit the int32 count", (long long)capacity);
    auto b = std::make_shared<Urb>();
    int rc = rows_alloc(b->rows, capacity, nfields, field_bytes);
    if (rc) return rc;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->err), 16 + kCntWords * sizeof(int64_t)));
    HIP_TRY(hipMemset(b->err, 0, 16 + kCntWords * sizeof(int64_t)));
    b->counters = reinterpret_cast<int64_t*>(b->err + 4);
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->slots), kUrbDrawMax * sizeof(int64_t)));
    HIP_TRY(hipDeviceSynchronize());  // the zero-fills ran on the null stream; the caller's stream may not wait for it
    std::lock_guard<std::mutex> lk(g_mu);
    *out_handle = g_next++;
    g_urb[*out_handle] = b;
    return MRB_OK;
}

int mrb_urb_append(int64_t h, const void* const* src_fields, int64_t nrows, void* stream) {
    GET_URB(b, h);
    if (nrows <= 0) return fail(MRB_EINVAL, "nrows %lld must be positive", (long long)nrows);
    const int64_t cap = b->rows.capacity;
    // Write position: `count` while the buffer has never wrapped, else `head` (the oldest row).
    const bool growing = b->count < cap && b->head == 0;
    const int64_t w = growing ? b->count : b->head;
    // More rows than slots: only the last `cap` survive, at the positions a row-by-row append leaves them.
    const int64_t skip = nrows > cap ? nrows - cap : 0;
    const int64_t first = (w + skip) % cap;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (b->device_counters) {
        // the write position is read on the device, and advanced there after the copy
        if (nrows > cap) return fail(MRB_ESTATE, "with device_counters an append takes at most capacity (%lld) rows", (long long)cap);
        PutArgs p{};
        int rc = put_args(b->rows, src_fields, 0, nrows, 0, p);
        if (rc) return rc;
        p.first_slot = -1;
        p.src_first = reinterpret_cast<int64_t>(b->counters);
        hipLaunchKernelGGL(k_rows_put, dim3(p.blocks), dim3(kWG), 0, s, p);
        LAUNCH_CHECK("k_rows_put");
        urb_advance(*b, nrows);
        return counters_advance(*b, nrows, 0, s);
    }
    int rc = rows_put(b->rows, src_fields, skip, nrows - skip, first, s);
    if (rc) return rc;
    urb_advance(*b, nrows);
    return MRB_OK;
}

/* Appends to `h` the `n` rows of uniform buffer `src` at logical positions first .. first + n - 1
 * (0 = oldest), in one launch. */
int mrb_urb_append_from(int64_t h, int64_t src, int64_t first_logical, int64_t n, void* stream) {
    GET_URB(b, h);
    auto from = find_urb(src);
    if (!from) return fail(MRB_EHANDLE, "unknown uniform buffer handle %lld", (long long)src);
    if (from.get() == b.get()) return fail(MRB_EINVAL, "source and destination are the same buffer");
    if (b->device_counters || from->device_counters)
        return fail(MRB_ESTATE, "a buffer-to-buffer append needs both buffers' counters on the host (device_counters 0)");
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (first_logical < 0) first_logical += from->count;
    if (first_logical < 0 || first_logical + n > from->count)
        return fail(MRB_EINVAL, "rows [%lld, %lld) outside the %lld stored rows", (long long)first_logical,
                    (long long)(first_logical + n), (long long)from->count);
    if (from->rows.nfields != b->rows.nfields) return fail(MRB_EINVAL, "buffers differ in their fields");
    for (int i = 0; i < b->rows.nfields; ++i)
        if (from->rows.bytes[i] != b->rows.bytes[i] || from->rows.stride[i] != b->rows.stride[i])
            return fail(MRB_EINVAL, "buffers differ in field %d (size or row layout)", i);
    const int64_t cap = b->rows.capacity;
    // source slot of the first row: logical -> physical as in get_item
    const int64_t t0 = from->count - from->head;
    const int64_t src_first = first_logical < t0 ? first_logical + from->head : first_logical - t0;
    const bool growing = b->count < cap && b->head == 0;
    const int64_t w = growing ? b->count : b->head;
    const int64_t skip = n > cap ? n - cap : 0;
    PutArgs p{};
    const void* io[MRB_MAX_FIELDS];
    for (int i = 0; i < b->rows.nfields; ++i) io[i] = from->rows.data[i];
    int rc = make_table(b->rows, io, n - skip, p.t);
    if (rc) return rc;
    p.capacity = cap;
    p.first_slot = (w + skip) % cap;
    p.src_capacity = from->rows.capacity;
    p.src_first = (src_first + skip) % from->rows.capacity;
    p.blocks = grid_for(p.t.prefix[p.t.nfields]);
    hipLaunchKernelGGL(k_rows_put, dim3(p.blocks), dim3(kWG), 0, static_cast<hipStream_t>(stream), p);
    LAUNCH_CHECK("k_rows_put");
    urb_advance(*b, n);
    return MRB_OK;
}

static int urb_gather_impl(Urb& b, const int64_t* indices, int64_t fixed_slot, int64_t n, int64_t* out_indices,
                           void* const* dst_fields, hipStream_t s) {
    return gather_rows(b.rows, indices, fixed_slot, b.count, b.seed, b.calls, n, out_indices, dst_fields, b.err, s);
}

int mrb_urb_get_item(int64_t h, int64_t logical_index, void* const* dst_fields, void* stream) {
    GET_URB(b, h);
    int64_t i = logical_index;
    if (i < 0) i += b->count;
    if (i < 0 || i >= b->count)
        return fail(MRB_EINVAL, "index %lld outside the %lld stored rows", (long long)logical_index, (long long)b->count);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (b->device_counters) {
        // count and head are read on the device: the slot is worked out there and the gather takes it as a given index
        hipLaunchKernelGGL(k_urb_slots, dim3(1), dim3(kWG), 0, s, b->slots, b->seed, b->counters, (int64_t)1, logical_index, 1,
                           b->err);
        LAUNCH_CHECK("k_urb_slots");
        return gather_rows(b->rows, b->slots, -1, b->rows.capacity, b->seed, b->calls, 1, nullptr, dst_fields, b->err, s);
    }
    const int64_t t = b->count - b->head;
    const int64_t slot = i < t ? i + b->head : i - t;
    return urb_gather_impl(*b, nullptr, slot, 1, nullptr, dst_fields, s);
}

int mrb_urb_gather(int64_t h, const int64_t* indices, int64_t n, void* const* dst_fields, void* stream) {
    GET_URB(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (!indices) return fail(MRB_EINVAL, "indices is NULL");
    if (b->count <= 0) return fail(MRB_ESTATE, "gather from an empty buffer");
    if (b->device_counters)  // the row count is on the device: slots are checked against the capacity only
        return gather_rows(b->rows, indices, -1, b->rows.capacity, b->seed, b->calls, n, nullptr, dst_fields, b->err,
                           static_cast<hipStream_t>(stream));
    return urb_gather_impl(*b, indices, -1, n, nullptr, dst_fields, static_cast<hipStream_t>(stream));
}

int mrb_urb_sample(int64_t h, int64_t n, int64_t* out_indices, void* const* dst_fields, void* stream) {
    GET_URB(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (n > b->count)
        return fail(MRB_ESTATE, "sample size %lld exceeds the %lld stored rows", (long long)n, (long long)b->count);
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (b->device_counters) {
        // count and the generator's call counter are read on the device: the slots are drawn there, the gather
        // takes them as given indices, and the call counter moves on there
        if (n > kUrbDrawMax)
            return fail(MRB_ESTATE, "with device_counters a sample takes at most %lld rows", (long long)kUrbDrawMax);
        hipLaunchKernelGGL(k_urb_slots, dim3(grid_exact((uint64_t)n)), dim3(kWG), 0, s, b->slots, b->seed, b->counters, n,
                           (int64_t)0, 0, b->err);
        LAUNCH_CHECK("k_urb_slots");
        int rc = gather_rows(b->rows, b->slots, -1, b->rows.capacity, b->seed, b->calls, n, out_indices, dst_fields, b->err, s);
        if (rc) return rc;
        b->calls += 1;
        return counters_advance(*b, 0, 1, s);
    }
    int rc = urb_gather_impl(*b, nullptr, -1, n, out_indices, dst_fields, s);
    if (rc) return rc;
    b->calls += 1;
    return MRB_OK;
}

int mrb_urb_seed(int64_t h, uint64_t seed) {
    GET_URB(b, h);
    if (b->device_counters) {
        const int rc = counters_from_device(*b);
        if (rc) return rc;
    }
    b->seed = seed;
    b->calls = 0;
    return b->device_counters ? counters_to_device(*b) : MRB_OK;
}

int mrb_urb_state(int64_t h, int32_t* count, int32_t* head) {
    GET_URB(b, h);
    if (b->device_counters) {  // the device's counters are the current ones (a graph replay advances only them)
        const int rc = counters_from_device(*b);
        if (rc) return rc;
    }
    if (count) *count = (int32_t)b->count;
    if (head) *head = (int32_t)b->head;
    return MRB_OK;
}

int mrb_urb_reset(int64_t h) {
    GET_URB(b, h);
    if (b->device_counters) {  // no stream to order it on: the counters come back, are reset and go out again
        int rc = counters_from_device(*b);
        if (rc) return rc;
        b->count = 0;
        return counters_to_device(*b);
    }
    b->count = 0;
    return MRB_OK;
}

int mrb_urb_check(int64_t h, uint32_t* flags, void* stream) {
    GET_URB(b, h);
    return read_and_clear_flags(b->err, flags, static_cast<hipStream_t>(stream));
}

int mrb_urb_field_ptr(int64_t h, int field, void** dev_ptr) {
    GET_URB(b, h);
    if (field < 0 || field >= b->rows.nfields || !dev_ptr) return fail(MRB_EINVAL, "bad field %d", field);
    *dev_ptr = b->rows.data[field];
    return MRB_OK;
}

int mrb_urb_destroy(int64_t h) {
    std::shared_ptr<Urb> b;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto it = g_urb.find(h);
        if (it == g_urb.end()) return fail(MRB_EHANDLE, "unknown uniform buffer handle %lld", (long long)h);
        b = it->second;
        g_urb.erase(it);
    }
    HIP_TRY(hipDeviceSynchronize());
    return MRB_OK;
}

/* ------------------------------------------------------------ prioritized */

int mrb_per_create(int64_t capacity, float alpha, int nfields, const int64_t* field_bytes, uint64_t seed,
                   int64_t* out_handle) {
    if (!out_handle) return fail(MRB_EINVAL, "out_handle is NULL");
    if (!(alpha >= 0.0f) || alpha > 16.0f) return fail(MRB_EINVAL, "alpha %g outside [0, 16]", (double)alpha);
    auto b = std::make_shared<Per>();
    int rc = rows_alloc(b->rows, capacity, nfields, field_bytes);
    if (rc) return rc;
    while (b->leaves < capacity) {
        b->leaves <<= 1;
        b->depth += 1;
    }
    b->alpha = alpha;
    b->seed = seed;
    // Rebuild plan: a tree of at most 12 levels is one workgroup's work (the top). A taller one gets as few
    // rounds (launches of a wave per 256-node tile) below its top as possible, and every round takes the full
    // 8 levels, which leaves the top - one workgroup, the end of every call's chain of launches - as low as
    // it can be: up to 8 levels it is one tile and one pass, beyond that tiles, a barrier and a second pass.
    b->top_depth = b->depth < kTopMaxDepth ? b->depth : kTopMaxDepth;
    if (const int rest = b->depth - b->top_depth; rest > 0) {
        // (21 levels: a top one level deeper, 32 tiles, saves a whole round, i.e. a launch)
        b->nrounds = rest == kRoundLevels + 1 ? 1 : (rest + kRoundLevels - 1) / kRoundLevels;
        b->top_depth = b->depth - kRoundLevels * b->nrounds;
    }
    for (int r = 0, lo = b->depth; r < b->nrounds; ++r) {
        b->lo[r] = lo;
        b->g[r] = kRoundLevels;
        lo -= kRoundLevels;
    }
    const size_t nodes = 2 * (size_t)b->leaves;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->sum), nodes * sizeof(float)));
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->mn), nodes * sizeof(float)));
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->stamp), (size_t)b->leaves * sizeof(unsigned long long)));
    // one allocation: the error word (16 bytes), the device copy of the counters (kernels find them behind the error
    // word), and kMaxpBehindErr bytes in the running max (16 bytes; a kernel that is given its address finds the
    // counters in front of it: counters_before)
    static_assert(16 + kCntWords * sizeof(int64_t) <= kMaxpBehindErr, "the counters end before the running max");
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->err), kMaxpBehindErr + 16));
    b->counters = reinterpret_cast<int64_t*>(b->err + 4);
    b->maxp = reinterpret_cast<float*>(reinterpret_cast<char*>(b->err) + kMaxpBehindErr);
    HIP_TRY(hipMemset(b->counters, 0, kCntWords * sizeof(int64_t)));
    // update_priorities scratch, sized once: a call rarely names more entries than there are rows
    b->powered_cap = capacity < 4096 ? 4096 : (capacity > (1ll << 20) ? (1ll << 20) : capacity);
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->powered), (size_t)b->powered_cap * sizeof(float)));
    HIP_TRY(hipGetDevice(&b->device));
    float* unused = nullptr;
    rc = static_scratch(&unused);  // set-up of the allocation-free entry point for this device
    if (rc) return rc;
    HIP_TRY(hipMemset(b->sum, 0, nodes * sizeof(float)));
    HIP_TRY(hipMemset(b->stamp, 0, (size_t)b->leaves * sizeof(unsigned long long)));
    HIP_TRY(hipMemset(b->err, 0, 16));
    for (int r = 0; r < b->nrounds; ++r) {
        const size_t nblocks = (size_t)1 << (b->lo[r] - b->g[r]);
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->dirty[r]), nblocks * sizeof(uint32_t)));
        HIP_TRY(hipMemset(b->dirty[r], 0, nblocks * sizeof(uint32_t)));
    }
    if (b->depth >= 22) {
        // sparse plan: with >= 16384 leaf tiles a call with few entries is better driven by its entries
        b->s_g0 = b->depth - 20 < 4 ? 4 : (b->depth - 20 > 6 ? 6 : b->depth - 20);
        const int d2 = b->depth - b->s_g0;
        b->s_top = kTopMaxDepth;
        const int rest2 = d2 - b->s_top;  // >= 4
        b->s_rounds = (rest2 + kRoundLevels - 1) / kRoundLevels;
        for (int r = 0, lo = d2; r < b->s_rounds; ++r) {
            b->s_lo[r] = lo;
            b->s_g[r] = rest2 / b->s_rounds + (r < rest2 % b->s_rounds ? 1 : 0);
            lo -= b->s_g[r];
            const size_t nblocks = (size_t)1 << (b->s_lo[r] - b->s_g[r]);
            HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->s_dirty[r]), nblocks * sizeof(uint32_t)));
            HIP_TRY(hipMemset(b->s_dirty[r], 0, nblocks * sizeof(uint32_t)));
        }
    }
    hipLaunchKernelGGL(k_fill_f32, dim3(grid_for(nodes)), dim3(kWG), 0, nullptr, b->mn, FLT_MAX, (uint64_t)nodes);
    LAUNCH_CHECK("k_fill_f32");
    const float one_then_zero[4] = {1.0f, 0.0f, 0.0f, 0.0f};  // the running max; the max a push in progress has seen
    HIP_TRY(hipMemcpy(b->maxp, one_then_zero, sizeof(one_then_zero), hipMemcpyHostToDevice));
    HIP_TRY(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lk(g_mu);
    *out_handle = g_next++;
    g_per[*out_handle] = b;
    return MRB_OK;
}

// The push behind mrb_per_push and mrb_per_update_push. `after_update`: an update_priorities of this very call
// precedes the push on the stream and changed nodes anywhere in the tree, so a one-launch push rebuilds the
// whole top (see UpdateArgs::full_top); `lead`, if given, is that update's leaf round, still to be launched:
// the push's row copy rides along in it and the push's own tree work follows as the last launch.
struct LeadRound {
    UpdateArgs a;
};

static int per_push(Per* b, const void* const* src_fields, int64_t nrows, const float* opt_priorities, hipStream_t s,
                    const LeadRound* lead = nullptr) {
    if (nrows <= 0) return fail(MRB_EINVAL, "nrows %lld must be positive", (long long)nrows);
    if (nrows > 0x7fffffffll) return fail(MRB_EINVAL, "nrows %lld exceeds 2^31 - 1 rows per call", (long long)nrows);
    const int64_t cap = b->rows.capacity;
    if (b->device_counters && nrows > cap)
        return fail(MRB_ESTATE, "with device_counters a push takes at most capacity (%lld) rows", (long long)cap);
    const int64_t skip = nrows > cap ? nrows - cap : 0;  // rows overwritten within this very call
    const int64_t n = nrows - skip;
    const int64_t first = (b->pushes + skip) % cap;
    PutArgs put{};
    int rc = put_args(b->rows, src_fields, skip, n, first, put);
    if (rc) return rc;
    if (b->device_counters) {  // the kernels take the first slot from the device
        put.first_slot = -1;
        put.src_first = reinterpret_cast<int64_t>(b->counters);
    }
    // A large copy gets its own launch; a small one rides along in the first tree launch.
    if (put.blocks > 2048u) {
        hipLaunchKernelGGL(k_rows_put, dim3(put.blocks), dim3(kWG), 0, s, put);
        LAUNCH_CHECK("k_rows_put");
        put.blocks = 0;
    }
    if (lead) {
        // the update's leaf round (a wave or two per entry), with this push's row copy as further workgroups
        const uint32_t waves = (lead->a.n > kPairedAbove ? 2u : 1u) * (uint32_t)lead->a.n;
        const UpdateArgs& la = lead->a;
        hipLaunchKernelGGL(k_tree_update, dim3((waves + 3) / 4 + put.blocks), dim3(kWG), 0, s, la.indices, la.priorities, la.sum,
                           la.mn, la.n, la.capacity, 0 | la.lo[0] << 8 | la.g[0] << 16, la.alpha, la, 0u, put);
        LAUNCH_CHECK("k_tree_update");
        put.blocks = 0;
    }
    rc = next_epoch(*b, s);
    if (rc) return rc;
    UpdateArgs a = update_args(*b);
    a.full_top = lead ? 1 : 0;
    // push-then-update: the running max sees every priority of the call, surviving or not, and is
    // raised only after the tree work (a fresh slot with an invalid priority keeps the old running max).
    // Few rows: the top workgroup scans the priorities itself. More: the leaf-level waves, which compute
    // every p^alpha anyway, collect their max beside the running max and the top workgroup folds it in.
    // Only a call that overwrites rows of its own (more rows than capacity) needs a pass over all priorities.
    const int fold = !opt_priorities ? 0 : (skip == 0 && nrows <= 1024) ? 1 : (skip == 0 && a.nrounds > 0) ? 2 : 0;
    if (opt_priorities) {
        a.priorities = opt_priorities + skip;
        a.fold_max = fold;
    }
    a.first_slot = b->device_counters ? -1 : first;
    a.n = n;
    a.advance = b->device_counters ? nrows : 0;  // the call's last launch moves the device's counters on
    const bool stamp_after = opt_priorities && !fold;
    if (!lead && b->fused && nrows == 1 && b->depth <= kPushOneMaxDepth) {
        // one row: one wave walks from its leaf to the root (k_push_one)
        rc = ride_alone_if_large(a, put, s);
        if (rc) return rc;
        hipLaunchKernelGGL(b->device_counters ? k_push_one<true> : k_push_one<false>, dim3(1 + put.blocks), dim3(kWG), 0, s,
                           a.sum, a.mn, a.maxp, a.first_slot, a.capacity, a.leaves, a.depth, a.alpha, opt_priorities, a.err, put,
                           a.advance, 1 + put.blocks * (kWG / 64));
        LAUNCH_CHECK("k_push_one");
        b->pushes += nrows;
        b->size = b->size + nrows < cap ? b->size + nrows : cap;
        return MRB_OK;
    }
    rc = tree_rebuild(*b, a, s, put.blocks ? &put : nullptr);
    if (rc) return rc;
    if (stamp_after) {
        a.priorities = opt_priorities;
        a.n = nrows;
        hipLaunchKernelGGL(k_update_stamp, dim3(grid_exact((uint64_t)nrows)), dim3(kWG), 0, s, a);
        LAUNCH_CHECK("k_update_stamp");
    }
    b->pushes += nrows;
    b->size = b->size + nrows < cap ? b->size + nrows : cap;
    return MRB_OK;
}

int mrb_per_push(int64_t h, const void* const* src_fields, int64_t nrows, const float* opt_priorities, void* stream) {
    GET_PER(b, h);
    return per_push(b.get(), src_fields, nrows, opt_priorities, static_cast<hipStream_t>(stream));
}

int mrb_per_update(int64_t h, const int64_t* indices, const float* priorities, int64_t n, void* stream) {
    GET_PER(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (n > 0xffffffffll) return fail(MRB_EINVAL, "n %lld exceeds 2^32 - 1 entries per call", (long long)n);
    if (!indices || !priorities) return fail(MRB_EINVAL, "indices or priorities is NULL");
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (n > b->powered_cap) {
        // more entries than any call so far (and than the capacity): a larger array, at least twice the
        // old one; the old one stays allocated, kernels already queued may still use it
        const int64_t want = n > 2 * b->powered_cap ? n : 2 * b->powered_cap;
        float* bigger = nullptr;
        HIP_TRY(hipMalloc(reinterpret_cast<void**>(&bigger), (size_t)want * sizeof(float)));
        if (b->powered) b->retired.push_back(b->powered);
        b->powered = bigger;
        b->powered_cap = want;
    }
    return per_update(*b, indices, priorities, n, b->powered, s);
}

int mrb_per_update_noalloc(int64_t h, const int64_t* indices, const float* priorities, int64_t n, void* stream) {
    GET_PER(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (n > kNoAllocMaxEntries)
        return fail(MRB_EINVAL, "n %lld exceeds the %lld entries the static scratch holds; use mrb_per_update",
                    (long long)n, (long long)kNoAllocMaxEntries);
    if (!indices || !priorities) return fail(MRB_EINVAL, "indices or priorities is NULL");
    float* powered = nullptr;
    int rc = static_scratch(&powered);
    if (rc) return rc;
    int dev = -1;
    HIP_TRY(hipGetDevice(&dev));
    if (dev != b->device) return fail(MRB_ESTATE, "the buffer lives on device %d, the current device is %d", b->device, dev);
    return per_update(*b, indices, priorities, n, powered, static_cast<hipStream_t>(stream));
}

// Leaf tiles a push of n rows can meet when its first slot is known (no wrap) or only known on the device.
static uint32_t push_tiles(const Per& b, int64_t first, int64_t n) {
    if (b.device_counters) {
        UpdateArgs t{};
        t.capacity = b.rows.capacity;
        t.n = n;
        return push_units(t);
    }
    if (first + n > b.rows.capacity) return 0xffffffffu;  // wraps: not a single run of tiles
    return (uint32_t)((first + n - 1) / kBlockNodes) - (uint32_t)(first / kBlockNodes) + 1;
}

int mrb_per_update_push(int64_t h, const int64_t* indices, const float* priorities, int64_t n,
                        const void* const* src_fields, int64_t nrows, const float* opt_push_priorities, void* stream) {
    GET_PER(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (n > 0xffffffffll) return fail(MRB_EINVAL, "n %lld exceeds 2^32 - 1 entries per call", (long long)n);
    if (!indices || !priorities) return fail(MRB_EINVAL, "indices or priorities is NULL");
    if (nrows <= 0) return fail(MRB_EINVAL, "nrows %lld must be positive", (long long)nrows);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cap = b->rows.capacity;
    const bool small_push = nrows <= cap && b->fused;
    // (1) one launch: the one-workgroup or one-wave update, then the walk of the one pushed row by the same workgroup
    const bool wg = n <= kWgBestEntries && b->depth >= 2 && b->depth <= kWgMaxDepth;
    const bool paths = n <= kPathEntries && b->depth <= kPathMaxDepth && b->depth >= 2;
    if (small_push && nrows == 1 && (wg || paths) && b->depth <= kPushOneMaxDepth) {
        if (!src_fields) return fail(MRB_EINVAL, "field pointer array is NULL");
        PutArgs put{};
        const int64_t first = b->pushes % cap;
        int rc = put_args(b->rows, src_fields, 0, 1, first, put);
        if (rc) return rc;
        if (b->device_counters) {
            put.first_slot = -1;
            put.src_first = reinterpret_cast<int64_t>(b->counters);
        }
        if (put.blocks <= (b->device_counters ? kRideWithCounters : 2048u)) {
            rc = next_epoch(*b, s);
            if (rc) return rc;
            UpdateArgs a = update_args(*b);
            a.indices = indices;
            a.priorities = priorities;
            a.n = n;
            a.advance = b->device_counters ? 1 : 0;
            const int64_t slot = b->device_counters ? -1 : first;
            // (readers: the waves that read the device's counters - the tree wave and every wave of the row copy)
            if (wg) {
                // (65 to 128 entries: 1024 threads, eight per entry - the kernel's one-step path below the staged top)
        const uint32_t threads = n > 64 && n <= 128 ? 1024u : n <= kWgMinThreads ? (uint32_t)kWgMinThreads : (uint32_t)((n + 63) / 64 * 64);
                a.readers = 1 + put.blocks * (threads / 64);
                hipLaunchKernelGGL(b->device_counters ? k_tree_wg_push<true> : k_tree_wg_push<false>, dim3(1 + put.blocks),
                                   dim3(threads), 0, s, a.indices, a.priorities, a.sum, a.mn, a.maxp, (int)a.n, a.depth,
                                   (int)a.capacity, a.alpha, a, slot, opt_push_priorities, put);
                LAUNCH_CHECK("k_tree_wg_push");
            } else {
                a.readers = 1 + put.blocks * (kWG / 64);
                hipLaunchKernelGGL(b->device_counters ? k_tree_paths_push<true> : k_tree_paths_push<false>, dim3(1 + put.blocks),
                                   dim3(kWG), 0, s, a, slot, opt_push_priorities, put);
                LAUNCH_CHECK("k_tree_paths_push");
            }
            b->pushes += 1;
            b->size = b->size + 1 < cap ? b->size + 1 : cap;
            return MRB_OK;
        }
    }
    // (2) two launches on a tree with one round of levels below its top: the update's leaf round with the push's
    // row copy riding along, then one workgroup that rebuilds the pushed slots' leaf tiles and the whole top
    if (small_push && b->nrounds == 1 && n <= kElectMax && n > kFusedWG / 64 && b->depth >= 2 &&
        push_tiles(*b, b->pushes % cap, nrows) <= (uint32_t)(kFusedWG / 64)) {
        int rc = next_epoch(*b, s);
        if (rc) return rc;
        LeadRound lead{update_args(*b)};
        lead.a.indices = indices;
        lead.a.priorities = priorities;
        lead.a.n = n;
        lead.a.inline_election = 1;
        return per_push(b.get(), src_fields, nrows, opt_push_priorities, s, &lead);
    }
    // (3) otherwise: the two calls, one after the other
    int rc = mrb_per_update(h, indices, priorities, n, stream);
    if (rc) return rc;
    return per_push(b.get(), src_fields, nrows, opt_push_priorities, s);
}

// `nbatch` batches of `batch` stratified samples each, as nbatch successive mrb_per_sample calls on
// an unchanged tree would draw them. Outputs hold nbatch * batch rows, batch after batch.
static int per_sample_impl(Per* b, int64_t nbatch, int64_t batch, float beta, const float* uniforms,
                           int64_t* out_indices, float* out_weights, void* const* out_fields, hipStream_t s,
                           const NextRows* next = nullptr) {
    if (batch <= 0 || batch > (1ll << 24)) return fail(MRB_EINVAL, "batch %lld outside [1, 2^24]", (long long)batch);
    if (nbatch <= 0 || nbatch > 4096 || nbatch * batch > (1ll << 24))
        return fail(MRB_EINVAL, "%lld batches of %lld rows exceed one call (at most 4096 batches, 2^24 rows)",
                    (long long)nbatch, (long long)batch);
    if (!out_indices || !out_weights) return fail(MRB_EINVAL, "out_indices or out_weights is NULL");
    if (b->size <= 0) return fail(MRB_ESTATE, "sample from an empty buffer");
    IoTable t;
    int rc = make_table(b->rows, out_fields, nbatch * batch, t);
    if (rc) return rc;
    SampleArgs a{};
    a.sum = b->sum;
    a.mn = b->mn;
    a.depth = b->depth;
    a.leaves = b->leaves;
    a.capacity = b->rows.capacity;
    a.size = b->size;
    a.batch = batch;
    a.beta = beta;
    a.uniforms = uniforms;
    a.seed = b->seed;
    a.calls = b->calls;
    a.out_idx = out_indices;
    a.out_w = out_weights;
    a.err = b->err;
    if (b->device_counters) {
        a.size = -1;  // the kernels take the number of stored rows from the device
        // the generator's call counter is on the device too: the kernels read it there and add the number of the
        // batch (see generator_calls)
        if (!uniforms) a.calls = 0;
    }
    const float* const draws = a.uniforms;  // the caller's, or NULL: the generator's, computed by the kernels
    const int64_t max_bytes = widest_field(b->rows);
    int path = (int)b->sample_path;
    if (path == 0) path = (batch >= 8192 && max_bytes <= 256) ? 2 : 1;
    if (next) {
        rc = sample_wide(b->rows, a, t, nbatch, s, next);  // always the wide-row kernel: the gathered field is wide
        if (rc) return rc;
    } else if (path == 1) {
        rc = sample_wide(b->rows, a, t, nbatch, s);
        if (rc) return rc;
    } else {
        // the LDS-top kernel takes one batch per launch (its batches are large enough to fill the chip)
        int levels = b->lds_levels > 0 ? (int)b->lds_levels : 9;
        if (levels > b->depth) levels = b->depth;
        const uint32_t ntop = (2u << levels) < 4 ? 4 : (2u << levels);
        const size_t lds = ntop * sizeof(float) + (kWG + 1) * sizeof(int64_t);
        for (int64_t i = 0; i < nbatch; ++i) {
            SampleArgs ai = a;
            IoTable ti = t;
            ai.uniforms = draws ? draws + i * batch : nullptr;
            ai.calls = a.calls + (uint64_t)i;
            ai.out_idx = out_indices + i * batch;
            ai.out_w = out_weights + i * batch;
            for (int f = 0; f < t.nfields; ++f) ti.io[f] = t.io[f] + (uint64_t)i * batch * t.row_bytes[f];
            hipLaunchKernelGGL(k_per_sample_lds, dim3((uint32_t)((batch + kWG - 1) / kWG)), dim3(kLdsWG), lds, s, ai.sum,
                               ai.uniforms, ai.mn, ai.depth, levels, (int)batch, beta, ai.seed, ai.calls, ai, ti);
            LAUNCH_CHECK("k_per_sample_lds");
        }
    }
    if (!uniforms) {
        b->calls += (uint64_t)nbatch;
        if (b->device_counters) return counters_advance(*b, 0, nbatch, s);
    }
    return MRB_OK;
}

int mrb_per_sample(int64_t h, int64_t batch, float beta, const float* uniforms, int64_t* out_indices,
                   float* out_weights, void* const* out_fields, void* stream) {
    GET_PER(b, h);
    return per_sample_impl(b.get(), 1, batch, beta, uniforms, out_indices, out_weights, out_fields,
                           static_cast<hipStream_t>(stream));
}

int mrb_per_sample_many(int64_t h, int64_t nbatch, int64_t batch, float beta, const float* uniforms,
                        int64_t* out_indices, float* out_weights, void* const* out_fields, void* stream) {
    GET_PER(b, h);
    return per_sample_impl(b.get(), nbatch, batch, beta, uniforms, out_indices, out_weights, out_fields,
                           static_cast<hipStream_t>(stream));
}

int mrb_per_update_push_sample(int64_t h, const int64_t* indices, const float* priorities, int64_t n,
                               const void* const* src_fields, int64_t nrows, const float* opt_push_priorities,
                               int64_t batch, float beta, const float* uniforms, int64_t* out_indices,
                               float* out_weights, void* const* out_fields, void* stream) {
    GET_PER(b, h);
    // (everything the three calls would refuse is refused before the first of them runs)
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (!indices || !priorities) return fail(MRB_EINVAL, "indices or priorities is NULL");
    if (nrows <= 0) return fail(MRB_EINVAL, "nrows %lld must be positive", (long long)nrows);
    if (!src_fields) return fail(MRB_EINVAL, "field pointer array is NULL");
    if (batch <= 0 || batch > (1ll << 24)) return fail(MRB_EINVAL, "batch %lld outside [1, 2^24]", (long long)batch);
    if (!out_indices || !out_weights) return fail(MRB_EINVAL, "out_indices or out_weights is NULL");
    IoTable t;
    int rc = make_table(b->rows, out_fields, batch, t);
    if (rc) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t cap = b->rows.capacity;
    // one launch of one workgroup: the update of at most 384 entries on a tree of at most 14 levels, one row, a batch
    // of at most a thread per stratum, and rows small enough for one workgroup to copy; the counters on the host
    if (b->fused && b->sample_path == 0 && nrows == 1 && n <= kWgBestEntries && b->depth >= 2 &&
        b->depth <= kWgMaxDepth && batch <= kStepThreads) {
        PutArgs put{};
        const int64_t first = b->pushes % cap;
        rc = put_args(b->rows, src_fields, 0, 1, first, put);
        if (rc) return rc;
        if (put.t.prefix[put.t.nfields] <= kStepMaxPut && t.prefix[t.nfields] <= kStepMaxGather) {
            rc = next_epoch(*b, s);
            if (rc) return rc;
            UpdateArgs a = update_args(*b);
            a.indices = indices;
            a.priorities = priorities;
            a.n = n;
            StepLate late{};
            late.err = b->err;
            late.priority = opt_push_priorities;
            late.uniforms = uniforms;
            late.out_idx = out_indices;
            late.out_w = out_weights;
            late.size = b->size + 1 < cap ? b->size + 1 : cap;  // as the push leaves it
            late.seed = b->seed;
            late.calls = b->calls;
            late.beta = beta;
            late.put = put.t;
            late.get = t;
            // (with device_counters the kernel takes the slot, the row count and the generator's call counter from the
            // device and moves them on itself)
            const bool wide = n > 64 && n <= 128;  // 1024 threads, eight per entry (see k_tree_wg)
            auto* const kernel = b->device_counters ? (wide ? k_tree_wg_push_sample<true, 1024> : k_tree_wg_push_sample<true, kStepThreads>)
                                                    : (wide ? k_tree_wg_push_sample<false, 1024> : k_tree_wg_push_sample<false, kStepThreads>);
            hipLaunchKernelGGL(kernel, dim3(1), dim3(wide ? 1024 : kStepThreads), 0, s, indices, priorities, b->sum, b->mn, a.maxp,
                               (int)(cap << 16 | (b->device_counters ? 0 : first)), (int)(n << 18 | batch << 8) | b->depth, a.alpha,
                               late);
            LAUNCH_CHECK("k_tree_wg_push_sample");
            b->pushes += 1;
            b->size = late.size;
            if (!uniforms) b->calls += 1;
            return MRB_OK;
        }
    }
    rc = mrb_per_update_push(h, indices, priorities, n, src_fields, nrows, opt_push_priorities, stream);
    if (rc) return rc;
    return per_sample_impl(b.get(), 1, batch, beta, uniforms, out_indices, out_weights, out_fields, s);
}

int mrb_per_sample_next(int64_t h, int64_t batch, float beta, const float* uniforms, int slot_field, int row_field,
                        int64_t* out_indices, float* out_weights, void* const* out_fields, void* out_next_rows,
                        void* stream) {
    GET_PER(b, h);
    const RowStore& r = b->rows;
    if (slot_field < 0 || slot_field >= r.nfields || r.bytes[slot_field] != 8)
        return fail(MRB_EINVAL, "slot_field %d must name a field of 8 bytes (one int64 slot number per row)", slot_field);
    if (row_field < 0 || row_field >= r.nfields || r.vec_log2[row_field] != 4)
        return fail(MRB_EINVAL, "row_field %d must name a field whose rows are multiples of 16 bytes", row_field);
    if (!out_next_rows) return fail(MRB_EINVAL, "out_next_rows is NULL");
    if (reinterpret_cast<uintptr_t>(out_next_rows) & 15u) return fail(MRB_EINVAL, "out_next_rows %p is not 16-byte aligned", out_next_rows);
    const NextRows next{slot_field, row_field, out_next_rows};
    return per_sample_impl(b.get(), 1, batch, beta, uniforms, out_indices, out_weights, out_fields,
                           static_cast<hipStream_t>(stream), &next);
}

int mrb_per_gather(int64_t h, const int64_t* indices, int64_t n, void* const* dst_fields, void* stream) {
    GET_PER(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (!indices) return fail(MRB_EINVAL, "indices is NULL");
    if (b->size <= 0) return fail(MRB_ESTATE, "gather from an empty buffer");
    return gather_rows(b->rows, indices, -1, b->size, 0, 0, n, nullptr, dst_fields, b->err,
                       static_cast<hipStream_t>(stream));
}

int mrb_per_export_tree(int64_t h, float* sum_heap, float* min_heap, int64_t* leaves, void* stream) {
    GET_PER(b, h);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t bytes = 2 * (size_t)b->leaves * sizeof(float);
    HIP_TRY(hipStreamSynchronize(s));
    if (sum_heap) HIP_TRY(hipMemcpy(sum_heap, b->sum, bytes, hipMemcpyDeviceToHost));
    if (min_heap) HIP_TRY(hipMemcpy(min_heap, b->mn, bytes, hipMemcpyDeviceToHost));
    if (leaves) *leaves = b->leaves;
    return MRB_OK;
}

int mrb_per_state(int64_t h, int64_t* size, int64_t* head, float* max_priority, void* stream) {
    GET_PER(b, h);
    if (b->device_counters) {  // the device's counters are the current ones (a graph replay advances only them)
        const int rc = counters_from_device(*b);
        if (rc) return rc;
    }
    if (size) *size = b->size;
    if (head) *head = b->pushes % b->rows.capacity;
    if (max_priority) {
        hipStream_t s = static_cast<hipStream_t>(stream);
        HIP_TRY(hipMemcpyAsync(max_priority, b->maxp, sizeof(float), hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    return MRB_OK;
}

int mrb_per_check(int64_t h, uint32_t* flags, void* stream) {
    GET_PER(b, h);
    return read_and_clear_flags(b->err, flags, static_cast<hipStream_t>(stream));
}

int mrb_per_field_ptr(int64_t h, int field, void** dev_ptr) {
    GET_PER(b, h);
    if (field < 0 || field >= b->rows.nfields || !dev_ptr) return fail(MRB_EINVAL, "bad field %d", field);
    *dev_ptr = b->rows.data[field];
    return MRB_OK;
}

int mrb_per_destroy(int64_t h) {
    std::shared_ptr<Per> b;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto it = g_per.find(h);
        if (it == g_per.end()) return fail(MRB_EHANDLE, "unknown priority buffer handle %lld", (long long)h);
        b = it->second;
        g_per.erase(it);
    }
    HIP_TRY(hipDeviceSynchronize());
    return MRB_OK;
}

/* -------------------------------------------------------------- reservoir */

int mrb_res_create(int64_t capacity, int nfields, const int64_t* field_bytes, uint64_t seed, int64_t* out_handle) {
    if (!out_handle) return fail(MRB_EINVAL, "out_handle is NULL");
    auto b = std::make_shared<Res>();
    int rc = rows_alloc(b->rows, capacity, nfields, field_bytes);
    if (rc) return rc;
    b->seed = seed;
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->stamp), (size_t)capacity * sizeof(unsigned long long)));
    HIP_TRY(hipMemset(b->stamp, 0, (size_t)capacity * sizeof(unsigned long long)));
    HIP_TRY(hipMalloc(reinterpret_cast<void**>(&b->err), 16));
    HIP_TRY(hipMemset(b->err, 0, 16));
    HIP_TRY(hipDeviceSynchronize());  // as in mrb_urb_create
    std::lock_guard<std::mutex> lk(g_mu);
    *out_handle = g_next++;
    g_res[*out_handle] = b;
    return MRB_OK;
}

int mrb_res_push(int64_t h, const void* const* src_fields, int64_t nrows, void* stream) {
    GET_RES(b, h);
    if (nrows <= 0) return fail(MRB_EINVAL, "nrows %lld must be positive", (long long)nrows);
    if (nrows > 0x7fffffffll) return fail(MRB_EINVAL, "nrows %lld exceeds 2^31 - 1 rows per call", (long long)nrows);
    hipStream_t s = static_cast<hipStream_t>(stream);
    IoTable t;
    int rc = make_table(b->rows, src_fields, nrows, t);
    if (rc) return rc;
    const int64_t cap = b->rows.capacity;
    // Rows of one call can only collide on a slot once replacement has begun.
    const bool elect = nrows > 1 && b->total + nrows > cap;
    if (elect) {
        b->epoch += 1;
        if ((uint32_t)b->epoch == 0) {
            // by a fill kernel, not a memset node: the caller may be capturing this stream
            fill_zero(b->stamp, (size_t)cap * sizeof(unsigned long long), s);
            LAUNCH_CHECK("k_fill_f32");
            b->epoch += 1;
        }
        hipLaunchKernelGGL(k_res_elect, dim3(grid_exact((uint64_t)nrows)), dim3(kWG), 0, s, b->stamp, b->total, nrows,
                           cap, b->seed, (uint32_t)b->epoch);
        LAUNCH_CHECK("k_res_elect");
    }
    hipLaunchKernelGGL(k_res_put, dim3(grid_for(t.prefix[t.nfields])), dim3(kWG), 0, s, t,
                       elect ? b->stamp : nullptr, b->total, cap, b->seed, (uint32_t)b->epoch);
    LAUNCH_CHECK("k_res_put");
    b->total += nrows;
    b->size = b->total < cap ? b->total : cap;
    return MRB_OK;
}

int mrb_res_sample(int64_t h, int64_t n, int64_t* out_indices, void* const* dst_fields, void* stream) {
    GET_RES(b, h);
    if (n <= 0) return fail(MRB_EINVAL, "n %lld must be positive", (long long)n);
    if (b->size <= 0) return fail(MRB_ESTATE, "sample from an empty buffer");
    int rc = gather_rows(b->rows, nullptr, -1, b->size, b->seed, b->calls + 1, n, out_indices, dst_fields, b->err,
                         static_cast<hipStream_t>(stream));
    if (rc) return rc;
    b->calls += 1;
    return MRB_OK;
}

int mrb_res_state(int64_t h, int64_t* size, int64_t* total) {
    GET_RES(b, h);
    if (size) *size = b->size;
    if (total) *total = b->total;
    return MRB_OK;
}

int mrb_res_field_ptr(int64_t h, int field, void** dev_ptr) {
    GET_RES(b, h);
    if (field < 0 || field >= b->rows.nfields || !dev_ptr) return fail(MRB_EINVAL, "bad field %d", field);
    *dev_ptr = b->rows.data[field];
    return MRB_OK;
}

int mrb_res_destroy(int64_t h) {
    std::shared_ptr<Res> b;
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto it = g_res.find(h);
        if (it == g_res.end()) return fail(MRB_EHANDLE, "unknown reservoir buffer handle %lld", (long long)h);
        b = it->second;
        g_res.erase(it);
    }
    HIP_TRY(hipDeviceSynchronize());
    return MRB_OK;
}

/* -------------------------------------------------------- checkpoint hooks */

int mrb_urb_get_counters(int64_t h, int64_t* out4) {
    GET_URB(b, h);
    if (!out4) return fail(MRB_EINVAL, "out4 is NULL");
    if (b->device_counters) {
        const int rc = counters_from_device(*b);
        if (rc) return rc;
    }
    out4[0] = b->count, out4[1] = b->head, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
    return MRB_OK;
}

int mrb_urb_set_counters(int64_t h, const int64_t* in4) {
    GET_URB(b, h);
    if (!in4) return fail(MRB_EINVAL, "in4 is NULL");
    const int64_t cap = b->rows.capacity;
    if (in4[0] < 0 || in4[0] > cap || in4[1] < 0 || in4[1] >= cap)
        return fail(MRB_EINVAL, "count %lld / head %lld do not fit capacity %lld", (long long)in4[0], (long long)in4[1],
                    (long long)cap);
    b->count = in4[0], b->head = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    return b->device_counters ? counters_to_device(*b) : MRB_OK;
}

int mrb_per_get_counters(int64_t h, int64_t* out4) {
    GET_PER(b, h);
    if (!out4) return fail(MRB_EINVAL, "out4 is NULL");
    if (b->device_counters) {
        const int rc = counters_from_device(*b);
        if (rc) return rc;
    }
    out4[0] = b->size, out4[1] = b->pushes, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
    return MRB_OK;
}

int mrb_per_set_counters(int64_t h, const int64_t* in4) {
    GET_PER(b, h);
    if (!in4) return fail(MRB_EINVAL, "in4 is NULL");
    const int64_t cap = b->rows.capacity;
    const int64_t want = in4[1] < cap ? in4[1] : cap;
    if (in4[1] < 0 || in4[0] != want)
        return fail(MRB_EINVAL, "size %lld does not follow from %lld pushes into capacity %lld", (long long)in4[0],
                    (long long)in4[1], (long long)cap);
    b->size = in4[0], b->pushes = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    return b->device_counters ? counters_to_device(*b) : MRB_OK;
}

int mrb_res_get_counters(int64_t h, int64_t* out4) {
    GET_RES(b, h);
    if (!out4) return fail(MRB_EINVAL, "out4 is NULL");
    out4[0] = b->size, out4[1] = b->total, out4[2] = (int64_t)b->seed, out4[3] = (int64_t)b->calls;
    return MRB_OK;
}

int mrb_res_set_counters(int64_t h, const int64_t* in4) {
    GET_RES(b, h);
    if (!in4) return fail(MRB_EINVAL, "in4 is NULL");
    const int64_t cap = b->rows.capacity;
    const int64_t want = in4[1] < cap ? in4[1] : cap;
    if (in4[1] < 0 || in4[0] != want)
        return fail(MRB_EINVAL, "size %lld does not follow from %lld rows pushed into capacity %lld", (long long)in4[0],
                    (long long)in4[1], (long long)cap);
    b->size = in4[0], b->total = in4[1], b->seed = (uint64_t)in4[2], b->calls = (uint64_t)in4[3];
    return MRB_OK;
}

int mrb_per_load_leaves(int64_t h, const float* leaves, int64_t n, float max_priority, void* stream) {
    GET_PER(b, h);
    if (n < 0 || n > b->rows.capacity) return fail(MRB_EINVAL, "n %lld outside [0, capacity]", (long long)n);
    if (n > 0 && !leaves) return fail(MRB_EINVAL, "leaves is NULL");
    if (!(max_priority >= 0.0f) || max_priority > 3.0e38f) return fail(MRB_EINVAL, "max_priority %g is not a priority", (double)max_priority);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t nodes = 2 * (size_t)b->leaves;
    fill_zero(b->sum, nodes * sizeof(float), s);
    hipLaunchKernelGGL(k_fill_f32, dim3(grid_for(nodes)), dim3(kWG), 0, s, b->mn, FLT_MAX, (uint64_t)nodes);
    LAUNCH_CHECK("k_fill_f32");
    hipLaunchKernelGGL(k_fill_f32, dim3(1), dim3(kWG), 0, s, b->maxp, max_priority, (uint64_t)1);
    LAUNCH_CHECK("k_fill_f32");
    if (n == 0) return MRB_OK;
    int rc = next_epoch(*b, s);
    if (rc) return rc;
    // a push of slots [0, n) whose priorities are taken as they are: x^1 == x exactly
    UpdateArgs a = update_args(*b);
    a.alpha = 1.0f;
    a.priorities = leaves;
    a.first_slot = 0;
    a.n = n;
    return tree_rebuild(*b, a, s);
}

/* ------------------------------------------------------------ measurement aids */

int mrb_bench_launch(int kind, void* dst, const void* src, int64_t bytes, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kind == 0) {
        hipLaunchKernelGGL(k_nothing, dim3(1), dim3(64), 0, s);
        LAUNCH_CHECK("k_nothing");
        return MRB_OK;
    }
    if (kind == 1) {
        if (!dst || !src || bytes <= 0) return fail(MRB_EINVAL, "copy of %lld bytes from %p to %p", (long long)bytes, src, dst);
        HIP_TRY(hipMemcpyDtoDAsync(dst, const_cast<void*>(src), (size_t)bytes, s));
        return MRB_OK;
    }
    return fail(MRB_EINVAL, "unknown kind %d", kind);
}

/* ------------------------------------------------------- discounted return */

int mrb_discounted_return(const float* reward, const uint8_t* done, const float* last_value, float* out,
                          int64_t timesteps, int64_t batch, int64_t inner, float gamma, void* stream) {
    if (!reward || !done || !last_value || !out) return fail(MRB_EINVAL, "a data pointer is NULL");
    if (timesteps <= 0 || batch <= 0 || inner <= 0)
        return fail(MRB_EINVAL, "timesteps %lld, batch %lld, inner %lld must be positive", (long long)timesteps,
                    (long long)batch, (long long)inner);
    if (!(gamma >= 0.0f && gamma <= 1.0f))
        return fail(MRB_EINVAL, "The discounted factor should be a number in range [0, 1], but got %g.", (double)gamma);
    const int64_t cols = batch * inner;
    if (cols > (1ll << 31) || cols > (1ll << 40) / timesteps)
        return fail(MRB_EINVAL, "%lld columns of %lld steps exceed one call (at most 2^31 columns, 2^40 elements)",
                    (long long)cols, (long long)timesteps);
    if (cols <= 256 * kDrCols) {
        // few columns (at most one 64-column tile per compute unit): a thread per column cannot keep
        // enough loads in flight; stage chunks through LDS
        hipLaunchKernelGGL(k_discounted_return_tiled, dim3((uint32_t)((cols + kDrCols - 1) / kDrCols)), dim3(kDrWG), 0,
                           static_cast<hipStream_t>(stream), reward, done, last_value, out, timesteps, batch, inner,
                           gamma);
        LAUNCH_CHECK("k_discounted_return_tiled");
        return MRB_OK;
    }
    hipLaunchKernelGGL(k_discounted_return, dim3(grid_exact((uint64_t)cols)), dim3(kWG), 0,
                       static_cast<hipStream_t>(stream), reward, done, last_value, out, timesteps, batch, inner, gamma);
    LAUNCH_CHECK("k_discounted_return");
    return MRB_OK;
}

}  // extern "C"
