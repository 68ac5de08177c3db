// HIP kernels of the replay-buffer library (gfx950, wave64). No MFMA: nothing
// here is a dense contraction; the row kernels are HBM copies and the tree
// kernels are latency/LDS work.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mrb.h"
#include "mrb_device.h"

namespace mrb {

constexpr int kWG = 256;          // threads per workgroup of the row and sample kernels
constexpr int kLdsWG = kWG + 64;  // the LDS-top sample kernel: kWG strata and a helper wave
constexpr int kRoundLevels = 8;   // most tree levels rebuilt by one round of k_tree_update
constexpr int kBlockNodes = 256;  // nodes per wave tile in k_tree_update (float4 per lane)
constexpr int kTopMaxDepth = 12;  // deepest level k_tree_top normally starts from (4096 nodes)

// Per-call table of the fields of a row, passed to kernels by value.
// `store` is the field's place in the buffer - row r of the field at store + r * stride: a [capacity, row_bytes]
// matrix of its own, or a column of the packed rows -, `io` the caller's contiguous [n, row_bytes] matrix
// (source of an append, destination of a gather).
struct IoTable {
    int nfields;
    uint8_t* store[MRB_MAX_FIELDS];
    uint8_t* io[MRB_MAX_FIELDS];
    uint32_t row_bytes[MRB_MAX_FIELDS];
    uint32_t stride[MRB_MAX_FIELDS];    // bytes from one row of the field to the next in `store`: row_bytes when every
                                        // field has an array of its own, the packed row's size when rows are packed
    uint32_t units[MRB_MAX_FIELDS];     // row_bytes >> vec_log2
    uint32_t vec_log2[MRB_MAX_FIELDS];  // copy granule: 16, 8, 4, 2 or 1 bytes
    uint64_t prefix[MRB_MAX_FIELDS + 1];  // running sum of n * units over fields
};

// Row pointers reach the kernels inside by-value tables, where the compiler cannot
// see that they point to global memory; the qualified type makes every row access a
// global_load/global_store rather than a flat one.
using gbyte = __attribute__((address_space(1))) uint8_t;
__device__ __forceinline__ gbyte* as_global(uint8_t* p) { return (gbyte*)p; }
__device__ __forceinline__ const gbyte* as_global(const uint8_t* p) { return (const gbyte*)p; }

// One granule of 1 << vl bytes. Rows are read once and written once, so both
// sides bypass the caches' retention (non-temporal).
__device__ __forceinline__ void copy_granule(gbyte* dst, const gbyte* src, uint32_t vl) {
    switch (vl) {
        case 4: {
            using v4 = __attribute__((ext_vector_type(4))) uint32_t;
            v4 t = __builtin_nontemporal_load((const __attribute__((address_space(1))) v4*)src);
            __builtin_nontemporal_store(t, (__attribute__((address_space(1))) v4*)dst);
            break;
        }
        case 3: {
            using v2 = __attribute__((ext_vector_type(2))) uint32_t;
            v2 t = __builtin_nontemporal_load((const __attribute__((address_space(1))) v2*)src);
            __builtin_nontemporal_store(t, (__attribute__((address_space(1))) v2*)dst);
            break;
        }
        case 2:
            *(__attribute__((address_space(1))) uint32_t*)dst = *(const __attribute__((address_space(1))) uint32_t*)src;
            break;
        case 1:
            *(__attribute__((address_space(1))) uint16_t*)dst = *(const __attribute__((address_space(1))) uint16_t*)src;
            break;
        default:
            *dst = *src;
            break;
    }
}

using granule_t = __attribute__((ext_vector_type(4))) uint32_t;  // one 16-byte copy granule

// One granule of 1 << vl bytes held between its load and its store. vl is wave-uniform; every size
// has its own member so that no value of one load is merged with another's (a merge would make the
// compiler wait for the load right away).
struct AnyGranule {
    granule_t q;
    uint64_t d;
    uint32_t w;
    uint16_t h;
    uint8_t b;
    __device__ __forceinline__ void load(const gbyte* src, uint32_t vl) {
        switch (vl) {
            case 4: q = *(const __attribute__((address_space(1))) granule_t*)src; break;
            case 3: d = *(const __attribute__((address_space(1))) uint64_t*)src; break;
            case 2: w = *(const __attribute__((address_space(1))) uint32_t*)src; break;
            case 1: h = *(const __attribute__((address_space(1))) uint16_t*)src; break;
            default: b = *src; break;
        }
    }
    __device__ __forceinline__ void store(gbyte* dst, uint32_t vl) const {
        switch (vl) {
            case 4: *(__attribute__((address_space(1))) granule_t*)dst = q; break;
            case 3: *(__attribute__((address_space(1))) uint64_t*)dst = d; break;
            case 2: *(__attribute__((address_space(1))) uint32_t*)dst = w; break;
            case 1: *(__attribute__((address_space(1))) uint16_t*)dst = h; break;
            default: *dst = b; break;
        }
    }
};

__device__ __forceinline__ int field_of(const IoTable& t, uint64_t w) {
    int f = 0;
    while (f + 1 < t.nfields && w >= t.prefix[f + 1]) ++f;
    return f;
}

__device__ __forceinline__ void split_work(uint64_t local, uint32_t units, uint64_t& row, uint32_t& unit) {
    if (local <= 0xffffffffull) {
        const uint32_t l32 = (uint32_t)local;
        const uint32_t r = l32 / units;
        row = r;
        unit = l32 - r * units;
    } else {
        row = local / units;
        unit = (uint32_t)(local - row * units);
    }
}

// ---------------------------------------------------------------------------
// Ring append: rows [0, nrows) of each io matrix go to slots
// (first_slot + row) mod capacity. Replaces P.BufferAppend
// (mindspore_rl/core/uniform_replay_buffer.py:82,114) and the row copy of
// PriorityReplayBufferPush (mindspore_rl/core/priority_replay_buffer.py:67-69).
// The host guarantees nrows <= capacity, so no two rows share a slot.
// ---------------------------------------------------------------------------
// src_capacity > 0: the source is itself a ring of that many rows and row r is read from its
// slot (src_first + r) mod src_capacity (buffer-to-buffer copy); 0: the source is contiguous.
struct PutArgs {
    IoTable t;
    int64_t capacity, first_slot, src_capacity, src_first;
    uint32_t blocks;  // workgroups doing this copy when it rides along in another kernel's launch (0: none)
    // first_slot < 0: the buffer's counters live on the device (see Counters below), the rows go to
    // (pushes mod capacity) onwards, and src_first - unused then, the source is never a ring - holds the
    // counters' address
};

// A prioritized buffer's counters as device memory, for callers that record their loop into a HIP
// graph: kernels then take the ring position, the number of stored rows and the generator's call
// counter from here, and a one-thread kernel advances them after each call, so that every replay
// continues where the one before stopped.
// Kernels are told through a negative first slot / row count in their arguments and find the counters
// behind the buffer's error word (one allocation: 16 bytes of flags, then the counters), so that the
// arguments of the ordinary case are what they were.
// ([3] counts the reports of a launch that moves the counters on; [4] is the ring position, pushes mod capacity, kept
// beside the count so that no kernel divides)
constexpr int kCntPushes = 0, kCntSize = 1, kCntCalls = 2, kCntPos = 4, kCntWords = 5;

__device__ __forceinline__ const int64_t* counters_behind(const uint32_t* err) {
    return reinterpret_cast<const int64_t*>(err + 4);
}
// A prioritized buffer's running max lives in the same allocation, kMaxpBehindErr bytes behind the error word: a
// kernel that has its address among its preloaded arguments finds the counters without reading another argument.
constexpr int kMaxpBehindErr = 64;
__device__ __forceinline__ int64_t* counters_before(float* maxp) {
    return reinterpret_cast<int64_t*>(reinterpret_cast<char*>(maxp) - kMaxpBehindErr + 16);
}
__device__ __forceinline__ int64_t ring_position(const int64_t* counters, int64_t capacity) {
    return counters[kCntPos];
}
// The counters after a push of `pushed` rows (at most `capacity`), stored.
__device__ __forceinline__ void counters_store_advanced(int64_t* counters, int64_t pushes, int64_t size, int64_t pos,
                                                        int64_t pushed, int64_t capacity) {
    counters[kCntPushes] = pushes + pushed;
    size += pushed;
    counters[kCntSize] = size < capacity ? size : capacity;
    pos += pushed;
    counters[kCntPos] = pos < capacity ? pos : pos - capacity;
}

// The generator's call counter for a sample kernel: the argument, or - when the counters live on the device (a
// negative row count tells) and the generator supplies the draws - the device's counter plus the argument (the
// number of the batch among those the call launches one by one).
__device__ __forceinline__ uint64_t generator_calls(const float* uniforms, uint64_t calls, int64_t size, const uint32_t* err) {
    if (uniforms || size >= 0) return calls;
    return (uint64_t)counters_behind(err)[kCntCalls] + calls;
}

// The counters as a wave found them, and what its report returned (see counters_report).
struct CounterTicket {
    int64_t pushes, size, pos;
    uint32_t before;  // reports ahead of this wave's
};
// (atomic loads: vector loads past the compute unit's caches, which wait for nothing but themselves)
__device__ __forceinline__ CounterTicket counters_take(const uint32_t* err) {
    const int64_t* counters = counters_behind(err);
    CounterTicket t;
    t.pushes = __hip_atomic_load(counters + kCntPushes, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    t.size = __hip_atomic_load(counters + kCntSize, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    t.pos = __hip_atomic_load(counters + kCntPos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    t.before = 0;
    return t;
}
__device__ __forceinline__ int64_t ticket_position(const CounterTicket& t, int64_t capacity) { return t.pos; }

// A push moves the device-resident counters on in its own last launch. Where that launch is also the one whose
// workgroups read the ring position (`readers` of them: the tree workgroup and the row copy's), every such
// workgroup reports here when it is done, and the last one to report advances the counters: no workgroup waits
// for another, and none can read a position already moved on. readers <= 1: the caller is the only reader left.
// Called by every thread of the workgroup (it contains a barrier); the counters' fourth word counts the reports.
// `known`: the counters as thread 0 took them when the kernel started (nobody changes them before this advance);
// without it thread 0 requests them here, ahead of the barrier and the report.
__device__ __forceinline__ void counters_push_done(uint32_t* err, int64_t pushed, int64_t capacity, uint32_t readers,
                                                   const CounterTicket* known = nullptr) {
    if (pushed <= 0) return;  // uniform over the launch
    CounterTicket t{};
    if (threadIdx.x == 0) t = known ? *known : counters_take(err);
    __syncthreads();  // every wave's reads of the position are behind it
    if (threadIdx.x != 0) return;
    int64_t* counters = reinterpret_cast<int64_t*>(err + 4);
    if (readers > 1) {
        unsigned int* arrived = reinterpret_cast<unsigned int*>(counters + 3);
        if (atomicAdd(arrived, 1u) != readers - 1) return;
        atomicExch(arrived, 0u);
    }
    counters_store_advanced(counters, t.pushes, t.size, t.pos, pushed, capacity);
}

// The same for the one-launch pushes whose tree work is a single wave (k_push_one, k_tree_wg_push,
// k_tree_paths_push), wave by wave and EARLY: what must precede the advance is every wave's READ of the
// counters, not its work. A wave takes the counters (counters_take: loads only), reports as soon as the values
// are there (counters_report: one atomic whose operand depends on the loaded values, so that it cannot be issued
// before they arrive; its result is not awaited here) and goes on with its work; when that is done it looks at
// what the atomic returned (counters_settle) and, if it was the last of the `readers` waves to report, stores the
// advanced counters, computed from the values it took - no load, and no round trip to L2 at the kernel's end.
// All three are called by whole waves; lane 0 acts. readers <= 1: the calling wave is the only reader.
__device__ __forceinline__ void counters_report(CounterTicket& t, uint32_t* err, uint32_t readers, uint32_t lane) {
    if (readers <= 1 || lane != 0) return;
    unsigned int* arrived = reinterpret_cast<unsigned int*>(reinterpret_cast<int64_t*>(err + 4) + 3);
    // (both counters are non-negative: the operand is 1)
    t.before = atomicAdd(arrived, 1u + (unsigned int)((uint64_t)(t.pushes | t.size | t.pos) >> 63));
}
__device__ __forceinline__ void counters_settle(const CounterTicket& t, uint32_t* err, int64_t pushed, int64_t capacity,
                                                uint32_t readers, uint32_t lane) {
    if (lane != 0) return;
    int64_t* counters = reinterpret_cast<int64_t*>(err + 4);
    if (readers > 1) {
        if (t.before != readers - 1) return;
        atomicExch(reinterpret_cast<unsigned int*>(counters + 3), 0u);
    }
    counters_store_advanced(counters, t.pushes, t.size, t.pos, pushed, capacity);
}

// How a workgroup that carries a row copy in another kernel's launch ends. The compiler lays such a kernel out as
// if the tree workgroup's code could follow the copy, and without the explicit wait it makes the tree workgroup
// wait, early on, for loads that only the copy ever issues (its first requests then go out one after the other
// instead of together: a third of a microsecond on a one-workgroup call).
__device__ __forceinline__ void rider_ends() {
    __builtin_amdgcn_s_waitcnt(0);
    __builtin_amdgcn_endpgm();
}

// The copy itself, by workgroup `block` of `nblocks` (grid-stride over the granules). known_first >= 0: the
// first slot, already read from the device's counters by the caller.
__device__ __forceinline__ void rows_put_part(const PutArgs& p, uint32_t block, uint32_t nblocks, int64_t known_first = -1) {
    const IoTable& t = p.t;
    const uint64_t total = t.prefix[t.nfields];
    const uint64_t stride = (uint64_t)nblocks * blockDim.x;
    const int64_t first_slot = known_first >= 0  ? known_first
                               : p.first_slot >= 0 ? p.first_slot
                                                   : ring_position(reinterpret_cast<const int64_t*>(p.src_first), p.capacity);
    for (uint64_t w = (uint64_t)block * blockDim.x + threadIdx.x; w < total; w += stride) {
        const int f = field_of(t, w);
        uint64_t row;
        uint32_t unit;
        split_work(w - t.prefix[f], t.units[f], row, unit);
        int64_t slot = first_slot + (int64_t)row;
        if (slot >= p.capacity) slot -= p.capacity;
        uint64_t src_row = row;
        if (p.src_capacity > 0) {
            int64_t q = p.src_first + (int64_t)row;
            if (q >= p.src_capacity) q -= p.src_capacity;
            src_row = (uint64_t)q;
        }
        const uint32_t vl = t.vec_log2[f];
        const uint64_t off = (uint64_t)unit << vl;
        // (a source that is itself a ring is another buffer's storage, laid out like this one's)
        copy_granule(as_global(t.store[f]) + (uint64_t)slot * t.stride[f] + off,
                     as_global(t.io[f]) + src_row * (p.src_capacity > 0 ? t.stride[f] : t.row_bytes[f]) + off, vl);
    }
}

__global__ __launch_bounds__(kWG) void k_rows_put(PutArgs p) { rows_put_part(p, blockIdx.x, gridDim.x); }

// ---------------------------------------------------------------------------
// Gather: io_f[k] = store_f[slot_k]. slot_k is `fixed_slot` when that is >= 0
// (single-row read), else comes from `indices` or, when that is NULL, from the
// counter-based generator (uniform in [0, count), with replacement). Replaces P.BufferSample / P.BufferGetItem
// (mindspore_rl/core/uniform_replay_buffer.py:83-89,128,139).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kWG) void k_rows_gather(IoTable t, int64_t capacity, int64_t count,
                                                     const int64_t* __restrict__ indices, int64_t fixed_slot,
                                                     uint64_t seed, uint64_t calls,
                                                     int64_t* __restrict__ out_indices,
                                                     uint32_t* __restrict__ err) {
    // blockIdx.y is the field: the table's entries for it are the same for every thread of the launch's row of
    // workgroups and come through scalar registers, requested with the other arguments. (Indexed by a field number
    // each thread works out for itself they were two more dependent trips to memory in a kernel that is a chain of
    // such trips and nothing else.)
    const int f = blockIdx.y;
    const uint32_t units = t.units[f], vl = t.vec_log2[f], row_bytes = t.row_bytes[f], stride_f = t.stride[f];
    const gbyte* const store = as_global(t.store[f]);
    gbyte* const io = as_global(t.io[f]);
    const uint64_t total = t.prefix[f + 1] - t.prefix[f];  // rows * units
    const uint64_t step = (uint64_t)gridDim.x * kWG;
    for (uint64_t w = (uint64_t)blockIdx.x * kWG + threadIdx.x; w < total; w += step) {
        uint64_t row;
        uint32_t unit;
        split_work(w, units, row, unit);
        int64_t slot = fixed_slot >= 0 ? fixed_slot : indices ? indices[row] : rng_below(seed, calls, row, count);
        // a fixed slot was range-checked by the host against the ring (it may lie above `count` after a reset)
        if (fixed_slot < 0 && (slot < 0 || slot >= count)) {
            if (f == 0 && unit == 0) atomicOr(err, MRB_DERR_INDEX);
            slot = slot < 0 ? 0 : (count > 0 ? count - 1 : 0);
            if (slot >= capacity) slot = capacity - 1;
        }
        if (out_indices && f == 0 && unit == 0) out_indices[row] = slot;
        const uint64_t off = (uint64_t)unit << vl;
        copy_granule(io + row * row_bytes + off, store + (uint64_t)slot * stride_f + off, vl);
    }
}

// ---------------------------------------------------------------------------
// Reservoir push (ReservoirReplayBufferPush,
// mindspore_rl/core/reservoir_replay_buffer.py:64,68-79), Algorithm R for a
// batch: row j of the call is row number t = total + j of the buffer's life.
//   t < capacity : slot t
//   otherwise    : r uniform in [0, t]; slot r if r < capacity, else dropped
// k_res_elect makes the last row of the call that picks a slot its owner
// (integer max of (epoch << 32 | j)); k_res_put copies the owners' rows.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int64_t reservoir_slot(int64_t t, int64_t capacity, uint64_t seed) {
    if (t < capacity) return t;
    const int64_t r = rng_below(seed, 0, (uint64_t)t, t + 1);
    return r < capacity ? r : -1;
}

__global__ __launch_bounds__(kWG) void k_res_elect(unsigned long long* __restrict__ stamp, int64_t total,
                                                   int64_t nrows, int64_t capacity, uint64_t seed, uint32_t epoch) {
    const int64_t j = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (j >= nrows) return;
    const int64_t slot = reservoir_slot(total + j, capacity, seed);
    if (slot >= 0) atomicMax(&stamp[slot], ((unsigned long long)epoch << 32) | (unsigned long long)j);
}

// stamp == NULL: a single row, no election needed.
__global__ __launch_bounds__(kWG) void k_res_put(IoTable t, const unsigned long long* __restrict__ stamp,
                                                 int64_t total, int64_t capacity, uint64_t seed, uint32_t epoch) {
    const uint64_t work = t.prefix[t.nfields];
    const uint64_t stride = (uint64_t)gridDim.x * kWG;
    for (uint64_t w = (uint64_t)blockIdx.x * kWG + threadIdx.x; w < work; w += stride) {
        const int f = field_of(t, w);
        uint64_t row;
        uint32_t unit;
        split_work(w - t.prefix[f], t.units[f], row, unit);
        const int64_t slot = reservoir_slot(total + (int64_t)row, capacity, seed);
        if (slot < 0) continue;
        if (stamp && stamp[slot] != (((unsigned long long)epoch << 32) | row)) continue;
        const uint32_t vl = t.vec_log2[f];
        const uint64_t off = (uint64_t)unit << vl;
        copy_granule(as_global(t.store[f]) + (uint64_t)slot * t.stride[f] + off,
                     as_global(t.io[f]) + row * t.row_bytes[f] + off, vl);
    }
}

// Arguments of a PER sample (the wide-row kernel takes what its tree walk needs as plain leading
// parameters instead).
struct SampleArgs {
    const float* sum;       // sum tree, heap order
    const float* uniforms;  // f32[batch] or NULL -> generator
    int64_t batch;
    int depth;              // log2(leaves)
    float beta;
    uint64_t seed, calls;
    int64_t leaves;
    int64_t capacity;
    int64_t size;           // rows stored; negative: read from the device (see Counters)
    const float* mn;        // min tree, heap order
    int64_t* out_idx;
    float* out_w;
    uint32_t* err;
};

// mass of stratum k: (u + k) * (total / batch), each operation rounded once.
__device__ __forceinline__ float stratum_mass(const SampleArgs& a, float total, int64_t k, float u) {
    const float seg = total / (float)a.batch;
    return (u + (float)k) * seg;
}
__device__ __forceinline__ float stratum_mass(const SampleArgs& a, float total, int64_t k) {
    return stratum_mass(a, total, k, a.uniforms ? a.uniforms[k] : rng_uniform(a.seed, a.calls, (uint64_t)k));
}

// w = (p / total * size)^-beta / (pmin / total * size)^-beta
__device__ __forceinline__ float is_weight(float p, float total, float pmin, float fsize, float beta) {
    const float max_w = powf_det(pmin / total * fsize, -beta);
    return powf_det(p / total * fsize, -beta) / max_w;
}

__device__ __forceinline__ void sample_flags(const SampleArgs& a, float total, int64_t idx, int64_t size) {
    if (!(total > 0.0f) || total > 3.0e38f) atomicOr(a.err, MRB_DERR_TOTAL);
    if (idx >= size) atomicOr(a.err, MRB_DERR_UNFILLED);
}

// ---------------------------------------------------------------------------
// Wide rows (at least one field of 1 KB or more): k_per_sample_wide (PER sample)
// and k_rows_gather_wide (gather at given / drawn / fixed slots).
//
// A row's fields are of two kinds: "wide" fields, whose rows are multiples of
// 16 bytes and are copied in 16-byte granules, and "narrow" fields (the
// others: scalars and short vectors), copied byte by byte. The granules
// (bytes) of each kind are numbered consecutively over the fields. `split` workgroups share a row (one unless a
// row has more than 2048 wide granules); workgroup `part` copies wide granules
// [part * share, (part + 1) * share), the row's first workgroup also the
// narrow ones. A workgroup is one "walker" wave and four copy waves:
//   walker   finds the row's slot - for a sample by walking the sum tree with
//            group_request / group_walk (one dependent load per 10 levels; the
//            first group sits under the root, so it is requested together with
//            the total and the uniform draw) - using nothing but kernel
//            arguments preloaded into scalar registers, and publishes it
//            through LDS. Afterwards it copies the narrow fields, computes the
//            importance weight (the two powers in two lanes of one instruction
//            stream) and writes index and weight, off the copy waves' path.
//   copy     meanwhile every copy thread works out where its up to kInF
//            granules lie within a row (field, offset, destination) from the
//            field table, and the first copy wave stages in LDS what the
//            walker needs afterwards (narrow-field table, output pointers,
//            the minimum priority). After the barrier one multiply-add per
//            granule gives the source address; all loads are issued before
//            the first store: a row costs one memory round trip, not one per
//            field.
// Everything read from the kernel-argument segment costs a memory round trip
// of its own when a kernel starts (nothing is cached across launches), which
// is why the walker touches none of it before the barrier and the copy waves
// fetch the table in one round.
// Sampling reads its rows non-temporally so that they do not push the tree
// out of the caches; the gathered batch is stored with ordinary stores (it is
// what the caller reads next).
// ---------------------------------------------------------------------------
struct WideField {  // one table entry, 32 bytes
    const uint8_t* src;  // the field's place in the buffer: row r at src + r * ss
    uint8_t* dst;        // the caller's [batch, row_bytes] matrix
    uint32_t rb;         // row_bytes
    uint32_t first;      // wide field: number of its first granule among the wide ones; narrow: of its first byte
    uint32_t ss;         // bytes from one row to the next in the buffer (row_bytes, or the packed row's size)
    uint32_t pad;
};
struct WidePlan {
    int split;              // workgroups per row
    uint32_t share;         // wide granules per workgroup
    uint32_t wide_items;    // wide granules per row
    uint32_t narrow_items;  // bytes of narrow fields per row
    int nwide, nnarrow;     // fields of each kind
    uint32_t nbatch;        // host side only: batches in the launch
    uint32_t pad;
    WideField f[MRB_MAX_FIELDS];  // the wide fields first, then the narrow ones
};

// What the walker of a sample needs after the descent.
struct SampleTail {
    const float* mn;  // min tree, heap order
    int64_t* out_idx;
    float* out_w;
    uint32_t* err;
    int64_t size;  // rows stored; negative: read from the device (see Counters)
    float beta;
};

constexpr int kCopyWaves = 4;
constexpr int kCopyThreads = 64 * kCopyWaves;
constexpr int kWideWG = 64 + kCopyThreads + 64;  // the walker wave, four copy waves and, for rows with narrow
                                                  // fields, a wave that carries those (launched only then)
constexpr int kMaxInFlight = 8;             // most granules a copy thread holds between its loads and its stores
constexpr int kFastWide = 2;                // wide fields whose table entries are fetched unconditionally, in one round

using g16 = __attribute__((address_space(1))) granule_t;

constexpr int kNarrowInF = 2;  // narrow bytes a thread of the first copy wave holds beside its wide granules

__device__ __forceinline__ uint32_t lane_u32(uint32_t x, int src_lane) {
    return (uint32_t)__builtin_amdgcn_readlane((int)x, src_lane);
}
__device__ __forceinline__ uint64_t lane_u64(uint64_t x, int src_lane) {
    return ((uint64_t)lane_u32((uint32_t)(x >> 32), src_lane) << 32) | lane_u32((uint32_t)x, src_lane);
}

// The narrow fields of a row, copied byte by byte by a wave of their own in the row's first
// workgroup (the sixth; a copy wave that also carried them would hold its wide stores back until
// the narrow loads have arrived: 0.06 us per launch of 512 Atari-shaped rows): lane l takes bytes l,
// l + 64, ... of the narrow fields' bytes, numbered consecutively over the fields. Narrow fields are small (scalars such as action, reward, done); byte
// granularity keeps their copy free of branches on a granule size.
struct NarrowWork {
    const gbyte* base[kNarrowInF];
    gbyte* dst[kNarrowInF];
    uint32_t rb[kNarrowInF];  // the byte's field: bytes from one row to the next in the buffer
    uint32_t live;  // bit j: position j holds a byte
    // the table entry of field `lane` (lanes 0 .. MRB_MAX_FIELDS - 1), kept for bytes past the first ones
    uint64_t e_src, e_dst;
    uint32_t e_rb, e_first, e_ss;

    // Each lane finds the fields of its bytes from the table's entries. Up to kNarrowFast narrow fields (the
    // usual few scalars) are read with wave-uniform indices - scalar loads, issued together, from lines of the
    // kernel-argument segment that the copy waves' own reads bring into the scalar cache. More fields than that:
    // lane q fetches entry q with one vector load (a round trip of its own through memory, which holds back the
    // workgroup's barrier when nothing else, such as a tree descent, takes as long) and the entries are read from
    // the lanes. Rows with more than 64 * kNarrowInF narrow bytes keep the per-lane copy for store().
    static constexpr int kNarrowFast = 4;
    __device__ __forceinline__ void take(const WidePlan& plan, int64_t k, uint32_t lane, uint64_t src_q, uint64_t dst_q,
                                         uint32_t rb_q, uint32_t first_q, uint32_t ss_q) {
#pragma unroll
        for (int j = 0; j < kNarrowInF; ++j) {
            const uint32_t rel = ((live >> j) & 1u ? lane + 64 * j : 0u) - first_q;  // wraps for bytes of earlier fields
            if (rel < rb_q) {
                base[j] = (const gbyte*)(src_q + rel);
                dst[j] = (gbyte*)(dst_q + rel);
                rb[j] = ss_q;
            }
        }
    }
    __device__ __forceinline__ void prepare(const WidePlan& plan, int64_t k, uint32_t lane) {
        live = 0;
#pragma unroll
        for (int j = 0; j < kNarrowInF; ++j) {
            base[j] = nullptr;
            dst[j] = nullptr;
            rb[j] = 0;
            if (lane + 64 * j < plan.narrow_items) live |= 1u << j;
        }
        e_src = e_dst = 0;
        e_rb = e_first = e_ss = 0;
        if (plan.nnarrow <= kNarrowFast && plan.narrow_items <= 64u * kNarrowInF) {  // wave-uniform
            WideField e[kNarrowFast];
#pragma unroll
            for (int i = 0; i < kNarrowFast; ++i) e[i] = plan.f[plan.nwide + (i < plan.nnarrow ? i : 0)];
#pragma unroll
            for (int i = 0; i < kNarrowFast; ++i)
                if (i < plan.nnarrow)
                    take(plan, k, lane, (uint64_t)e[i].src, (uint64_t)e[i].dst + (uint64_t)k * e[i].rb, e[i].rb, e[i].first, e[i].ss);
            return;
        }
        const WideField e = plan.f[lane < MRB_MAX_FIELDS ? lane : 0];
        e_src = (uint64_t)e.src;
        e_dst = (uint64_t)e.dst + (uint64_t)k * e.rb;
        e_rb = e.rb;
        e_first = e.first;
        e_ss = e.ss;
        for (int q = plan.nwide; q < plan.nwide + plan.nnarrow; ++q)
            take(plan, k, lane, lane_u64(e_src, q), lane_u64(e_dst, q), lane_u32(e_rb, q), lane_u32(e_first, q), lane_u32(e_ss, q));
    }
    __device__ __forceinline__ void load(uint32_t slot, uint8_t (&held)[kNarrowInF]) const {
#pragma unroll
        for (int j = 0; j < kNarrowInF; ++j) held[j] = *(base[j] + (uint64_t)slot * rb[j]);
    }
    __device__ __forceinline__ void store(uint32_t slot, const uint8_t (&held)[kNarrowInF], const WidePlan& plan, uint32_t lane) const {
#pragma unroll
        for (int j = 0; j < kNarrowInF; ++j)
            if (live & (1u << j)) *dst[j] = held[j];
        if (plan.narrow_items > 64u * kNarrowInF) {  // wave-uniform; rows with many narrow bytes
            for (int q = plan.nwide; q < plan.nwide + plan.nnarrow; ++q) {
                const uint64_t src_q = lane_u64(e_src, q) + (uint64_t)slot * lane_u32(e_ss, q), dst_q = lane_u64(e_dst, q);
                const uint32_t rb_q = lane_u32(e_rb, q), first_q = lane_u32(e_first, q);
                // bytes of this field numbered 64 * kNarrowInF or more among the narrow bytes
                uint32_t rel = (first_q >= 64u * kNarrowInF ? 0u : 64u * kNarrowInF - first_q) + lane;
                for (; rel < rb_q; rel += 64) *((gbyte*)dst_q + rel) = *((const gbyte*)src_q + rel);
            }
        }
    }
};

// Copy thread `tid` (0 .. kCopyThreads - 1) of workgroup `part` of row k: up to kInF wide granules.
// A thread without a granule in some position re-reads the workgroup's first granule (a valid
// address) and skips the store, so that the loads are unconditional and all in flight together.
// kOneWide: the row has a single wide field (e.g. an image observation beside a few scalars); all
// addresses are then a wave-uniform row base plus a 32-bit offset, which costs a tenth of the
// general path's address arithmetic - work that would otherwise compete with the walker for
// the SIMD's issue slots.
// kThreads: the threads that share a workgroup's granules (the four copy waves; one wave in k_per_sample_rows).
template <int kInF, bool kOneWide, int kThreads = kCopyThreads>
struct CopyWork {
    const gbyte* base[kOneWide ? 1 : kInF];  // general: field storage + offset of the granule within a row
    g16* dst[kOneWide ? 1 : kInF];
    uint32_t rb[kOneWide ? 1 : kInF];        // general: bytes from one row to the next in the buffer
    uint32_t off[kOneWide ? kInF : 1];       // one wide field: byte offset of the granule within a row
    const uint8_t* src0;                     // one wide field: storage, destination row, storage row stride (wave-uniform)
    uint8_t* dst0;
    uint32_t rb0;
    uint32_t live;  // bit j: position j holds a granule of this workgroup

    __device__ __forceinline__ void prepare(const WidePlan& plan, int64_t k, uint32_t part, uint32_t tid) {
        const uint32_t lo = part * plan.share;
        const uint32_t hi = min(plan.wide_items, lo + plan.share);
        uint32_t it[kInF];
        live = 0;
#pragma unroll
        for (int j = 0; j < kInF; ++j) {
            it[j] = lo + j * kThreads + tid;
            if (it[j] < hi) live |= 1u << j;
            else it[j] = lo;
        }
        if (lo >= hi || tid >= (uint32_t)kThreads) live = 0;  // (a wave past the copy waves carries narrow fields only)
        if (kOneWide) {
            const WideField e = plan.f[0];
            src0 = e.src;
            rb0 = e.ss;
            dst0 = e.dst + (uint64_t)k * e.rb;
#pragma unroll
            for (int j = 0; j < kInF; ++j) off[j] = it[j] << 4;
            return;
        }
#pragma unroll
        for (int j = 0; j < (kOneWide ? 1 : kInF); ++j) {
            base[j] = nullptr;
            dst[j] = nullptr;
            rb[j] = 0;
        }
        auto take = [&](int q) {
            const WideField e = plan.f[q];
            const uint32_t units = q < plan.nwide ? e.rb >> 4 : 0u;
            const gbyte* s = as_global(e.src);
            gbyte* d = as_global(e.dst) + (uint64_t)k * e.rb;
#pragma unroll
            for (int j = 0; j < (kOneWide ? 1 : kInF); ++j) {
                const uint32_t rel = it[j] - e.first;  // wraps for granules of earlier fields
                if (rel < units) {
                    base[j] = s + ((uint64_t)rel << 4);
                    dst[j] = (g16*)(d + ((uint64_t)rel << 4));
                    rb[j] = e.ss;
                }
            }
        };
        // the first entries unconditionally: their (wave-uniform) loads go out together at once
#pragma unroll
        for (int q = 0; q < kFastWide; ++q) take(q);
        for (int q = kFastWide; q < plan.nwide; ++q) take(q);
    }

    // `narrow`: this thread carries narrow bytes (the wave after the copy waves, in the row's first workgroup)
    __device__ __forceinline__ void run(uint32_t slot, const WidePlan& plan, bool narrow, const NarrowWork& nw, uint32_t lane) const {
        uint8_t nheld[kNarrowInF];
        granule_t held[kInF];
        if (narrow) nw.load(slot, nheld);
        if (live) {
            if (kOneWide) {
                const gbyte* row = as_global(src0) + (uint64_t)slot * rb0;  // wave-uniform
#pragma unroll
                for (int j = 0; j < kInF; ++j) held[j] = __builtin_nontemporal_load((const g16*)(row + off[j]));
            } else {
#pragma unroll
                for (int j = 0; j < kInF; ++j)
                    held[j] = __builtin_nontemporal_load((const g16*)(base[j < (kOneWide ? 1 : kInF) ? j : 0] + (uint64_t)slot * rb[j < (kOneWide ? 1 : kInF) ? j : 0]));
            }
            // every load is issued before the first store (the compiler would otherwise move a load
            // next to its conditional store, behind the other stores' waits)
#pragma unroll
            for (int j = 0; j < kInF; ++j) asm volatile("" : "+v"(held[j]));
#pragma unroll
            for (int j = 0; j < kInF; ++j) {
                if (live & (1u << j)) {
                    if (kOneWide) *(g16*)(as_global(dst0) + off[j]) = held[j];
                    else *dst[j < (kOneWide ? 1 : kInF) ? j : 0] = held[j];
                }
            }
        }
        if (narrow) nw.store(slot, nheld, plan, lane);
    }
};

// Replaces PriorityReplayBufferSample (mindspore_rl/core/priority_replay_buffer.py:70,92-106).
// sum .. calls are the arguments the tree walk needs; they are preloaded into scalar registers.
// `groups` packs the descent plan: bits 0-3 the number of node groups, then 5 bits per group
// with the levels it takes; bits 20-31 hold the number of batches in the launch minus one. kTen: every group takes 10 levels (trees of 10, 20 or 30 levels); the
// walk is then compiled for that size, which shortens it by a third.
//
// kNext (k_per_sample_next): the launch has a second layer of workgroups (blockIdx.z == 1) that gathers, for
// every sampled row, ONE wide field at the slot the row itself names in an 8-byte field - the next observation
// of a transition that stores a slot number instead of a copy (`nx`). Such a workgroup repeats the walk, reads
// the slot number from the sampled row, and its copy waves copy that field's row; one launch then pays the
// launch and the descent for twice the bytes.
struct NextPlan {
    const uint8_t* slot_field;  // the 8-byte field that holds the slot number: row r at slot_field + r * slot_stride
    uint32_t slot_stride;
    WidePlan plan;              // one wide field: its storage -> the caller's [batch, row_bytes] matrix
};

struct NoNext {};

// kCW: copy waves of a workgroup (four; two in k_per_sample_light, for rows of at most 4 KB).
template <int kInF, bool kTen, bool kOneWide, bool kNext, typename Next, int kCW = kCopyWaves>
__device__ __forceinline__ void sample_wide_body(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                 int depth, uint32_t groups, int batch, uint32_t capacity,
                                                 uint64_t seed, uint64_t calls, const SampleTail& tail,
                                                 const WidePlan& plan, const Next& nx) {
    // the next-slot layer's plan and slot field (the row's own plan stands in where there is no such layer)
    const WidePlan& plan2 = [&]() -> const WidePlan& {
        if constexpr (kNext) return nx.plan;
        else return plan;
    }();
    const uint8_t* const slot_field = [&]() -> const uint8_t* {
        if constexpr (kNext) return nx.slot_field;
        else return nullptr;
    }();
    const uint32_t slot_stride = [&]() -> uint32_t {
        if constexpr (kNext) return nx.slot_stride;
        else return 8u;
    }();
    __shared__ int64_t s_idx;
    __shared__ float s_picked, s_total, s_pmin;
    __shared__ float s_tot[4];
    __shared__ SampleTail s_tail;
    const int64_t k = blockIdx.x;      // output row
    const uint32_t part = blockIdx.y;  // which of the row's workgroups
    const bool next_layer = kNext && blockIdx.z == 1;  // this workgroup gathers the row's next-slot field
    if (kNext && part >= (uint32_t)(next_layer ? plan2.split : plan.split)) return;  // the layers' splits may differ
    // Several batches in one launch (groups >> 20 = their number - 1): output row k is stratum `stratum`
    // of batch `nth`; each batch is stratified on its own and takes the generator's next call counter.
    uint32_t stratum = (uint32_t)k, nth = 0;
    if (groups >> 20) {
        nth = (uint32_t)k / (uint32_t)batch;
        stratum = (uint32_t)k - nth * (uint32_t)batch;
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool walker = wave == 0;
    const bool deep = depth == 21 || depth == 22;
    const uint32_t ctid = threadIdx.x - 64;  // copy thread number

    if (deep) {
        // Trees of 21 and 22 levels would need three dependent node groups of <= 10 levels. Instead
        // two (four) copy waves share the 2048 (4096) nodes at depth 11 (12), whose address is known: each
        // reduces its 1024 nodes, the wave totals - the tree's nodes at depth 1 (2) - meet in LDS, every
        // wave takes the one (two) top steps of the walk from them, and the wave the walk enters goes on
        // through its ten levels and the ten below. Two dependent loads again, one barrier more.
        const int share = depth - 20;  // log2 of the waves sharing the top group
        const int w = wave - 1;
        const bool mine = !walker && w < (1 << share);
        f32x4 r0, r1, r2, r3;
        f32x16 v = 0.0f;
        float total = 0.0f, u = 0.0f;
        if (mine) {
            group_request(sum, (1u << share) + w, kGroupMaxLevels, lane, r0, r1, r2, r3);
            total = sum[1];
            const uint64_t calls_now = generator_calls(uniforms, calls, tail.size, tail.err);
            u = uniforms ? uniforms[k] : rng_uniform(seed, calls_now + nth, (uint64_t)stratum);
            __builtin_amdgcn_sched_barrier(0);
            v = group_finish(kGroupMaxLevels, lane, r0, r1, r2, r3);
            const float t = group_total(v);
            if (lane == 0) s_tot[w] = t;
        }
        __syncthreads();
        if (mine) {
            float mass = (u + (float)stratum) * (total / (float)batch);  // each operation rounded once
            uint32_t q = 0;
            if (share == 2) {
                const float left = s_tot[0] + s_tot[1];  // the node at depth 1
                if (!(mass <= left)) {
                    mass -= left;
                    q = 2;
                }
            }
            const float left = s_tot[q];
            if (!(mass <= left)) {
                mass -= left;
                q += 1;
            }
            if ((uint32_t)w == q) {
                float picked;
                uint32_t node = (((1u << share) + q) << kGroupMaxLevels) + group_walk(v, kGroupMaxLevels, lane, mass, picked);
                group_request(sum, node, kGroupMaxLevels, lane, r0, r1, r2, r3);
                __builtin_amdgcn_sched_barrier(0);
                node = (node << kGroupMaxLevels) +
                       group_walk(group_finish(kGroupMaxLevels, lane, r0, r1, r2, r3), kGroupMaxLevels, lane, mass, picked);
                if (lane == 0) {
                    s_idx = (int64_t)node - ((int64_t)1 << depth);
                    s_picked = picked;
                    s_total = total;
                }
            }
        }
    } else if (walker) {
        // the walk is a chain of dependent instructions: it goes ahead of the copy waves' address
        // arithmetic on the SIMD they share
        __builtin_amdgcn_s_setprio(3);
        const int ngroups = (int)(groups & 15u);  // (bits 4-18: the groups' sizes, bits 20-31: batches - 1)
        uint32_t node = 1;
        float picked, mass = 0.0f, total;
        if (depth >= 2) {
            // The first group hangs under the root: its address is known, so it is requested at once,
            // together with the total and the draw (read from a valid address also when the generator
            // supplies the draw: no branch sits between the requests); the scheduling barrier keeps
            // every request ahead of the first use and of the generator's arithmetic.
            uint32_t packed = (groups >> 4) & 0x7fffu;
            int g = kTen ? kGroupMaxLevels : (int)(packed & 31u);
            f32x4 r0, r1, r2, r3;
            group_request(sum, 1u, g, lane, r0, r1, r2, r3);
            // (vector loads, through an offset the compiler cannot see through: as scalar loads they would be waited
            // for together with the reads of the kernel-argument segment that the other waves' code begins with)
            uint32_t opaque_zero = 0;
            asm volatile("" : "+v"(opaque_zero));
            total = sum[1 + opaque_zero];
            const float u_given = (uniforms ? uniforms + k : sum + 1)[opaque_zero];
            uint64_t calls_now = calls;
            if (!uniforms && (groups & (1u << 19))) calls_now += (uint64_t)counters_behind(tail.err)[kCntCalls];
            __builtin_amdgcn_sched_barrier(0);
            const float u = uniforms ? u_given : rng_uniform(seed, calls_now + nth, (uint64_t)stratum);
            mass = (u + (float)stratum) * (total / (float)batch);  // each operation rounded once
            node = (1u << g) + group_walk(group_finish(g, lane, r0, r1, r2, r3), g, lane, mass, picked);
#pragma nounroll
            for (int i = 1; i < ngroups; ++i) {
                packed >>= 5;
                g = kTen ? kGroupMaxLevels : (int)(packed & 31u);
                group_request(sum, node, g, lane, r0, r1, r2, r3);
                __builtin_amdgcn_sched_barrier(0);
                node = (node << g) + group_walk(group_finish(g, lane, r0, r1, r2, r3), g, lane, mass, picked);
            }
        } else {
            // one or two leaves
            total = sum[1];
            const float u = uniforms ? uniforms[k] : rng_uniform(seed, generator_calls(uniforms, calls, tail.size, tail.err) + nth, (uint64_t)stratum);
            mass = (u + (float)stratum) * (total / (float)batch);
            picked = total;
            node = (1u << depth) + (depth ? group_walk(group_load_tiny(sum, 1u, depth, lane), depth, lane, mass, picked) : 0u);
        }
        if (lane == 0) {
            s_idx = (int64_t)node - ((int64_t)1 << depth);
            s_picked = picked;
            s_total = total;
        }
        __builtin_amdgcn_s_setprio(0);
    }
    // ---- copy waves, while the walker walks
    CopyWork<kInF, kOneWide, 64 * kCW> work;
    NarrowWork nw;
    const bool narrow = wave == 1 + kCW && part == 0 && plan.narrow_items && !next_layer;
    if (!walker) {
        if (narrow) nw.prepare(plan, k, lane);
        if (next_layer) work.prepare(plan2, k, part, ctid);
        else work.prepare(plan, k, part, ctid);
        if ((part == 0 || next_layer) && wave == 2) {
            // what the walker needs after the barrier (member by member: a whole-struct copy would go
            // through private memory)
            if (lane == 0) {
                s_tail.out_idx = tail.out_idx;
                s_tail.out_w = tail.out_w;
                s_tail.err = tail.err;
                // (device-resident counters, see Counters: the number of stored rows is fetched here, beside the walk)
                s_tail.size = tail.size >= 0 ? tail.size : counters_behind(tail.err)[kCntSize];
                s_tail.beta = tail.beta;
            } else if (lane == 1) {
                s_pmin = tail.mn[1];
            }
        }
    }
    __syncthreads();
    const int64_t idx = s_idx;
    if (kNext && next_layer) {
        // the slot the sampled row names (outside [0, size): clamped and flagged, as mrb_per_gather does)
        __shared__ int64_t s_next;
        if (walker && lane == 0) {
            const int64_t size = s_tail.size;
            const int64_t row = idx < (int64_t)capacity ? idx : (int64_t)capacity - 1;
            int64_t to = *reinterpret_cast<const int64_t*>(slot_field + (uint64_t)row * slot_stride);
            if (to < 0 || to >= size) {
                if (part == 0) atomicOr(s_tail.err, MRB_DERR_INDEX);
                to = to < 0 ? 0 : (size > 0 ? size - 1 : 0);
            }
            s_next = to;
        }
        __syncthreads();
        if (!walker) work.run((uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)s_next), plan2, false, nw, lane);
        return;
    }
    if (!walker) {
        // the descent can end on an unfilled leaf past the last row (flagged by the walker)
        const uint32_t slot = (uint32_t)(idx < (int64_t)capacity ? idx : (int64_t)capacity - 1);
        work.run((uint32_t)__builtin_amdgcn_readfirstlane((int)slot), plan, narrow, nw, lane);
        return;
    }
    // ---- walker of the row's first workgroup: index and importance weight
    if (part != 0) return;
    // lane 0: (p / total * size)^-beta, lane 1: (pmin / total * size)^-beta
    const float total = s_total;
    const int64_t size = s_tail.size;
    const float fsize = (float)size;
    const float x = lane == 0 ? s_picked : s_pmin;
    float r = 0.0f;
    if (lane < 2) r = powf_det_call(x / total * fsize, -s_tail.beta);
    const float max_w = __shfl(r, 1);
    if (lane == 0) {
        s_tail.out_idx[k] = idx;
        s_tail.out_w[k] = r / max_w;
        if (!(total > 0.0f) || total > 3.0e38f) atomicOr(s_tail.err, MRB_DERR_TOTAL);
        if (idx >= size) atomicOr(s_tail.err, MRB_DERR_UNFILLED);
    }
}

template <int kInF, bool kTen, bool kOneWide>
__global__ __launch_bounds__(kWideWG) void k_per_sample_wide(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                             int depth, uint32_t groups, int batch, uint32_t capacity,
                                                             uint64_t seed, uint64_t calls, SampleTail tail, WidePlan plan) {
    sample_wide_body<kInF, kTen, kOneWide, false>(sum, uniforms, depth, groups, batch, capacity, seed, calls, tail, plan, NoNext{});
}

// The same kernel with two copy waves instead of four, for rows of at most 4 KB in 16-byte fields (two granules per
// copy thread): a workgroup of three or four waves per row instead of five or six. Rows that small leave most of
// four copy waves idle, and a launch of a thousand of them is bound by the number of waves to dispatch (config 4,
// 1024 rows of 521 B). Trees of 22 levels, whose walk four copy waves share, keep the full kernel.
constexpr int kLightCopyWaves = 2;
constexpr int kLightWG = 64 + 64 * kLightCopyWaves + 64;
template <bool kTen, bool kOneWide>
__global__ __launch_bounds__(kLightWG) void k_per_sample_light(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                               int depth, uint32_t groups, int batch, uint32_t capacity,
                                                               uint64_t seed, uint64_t calls, SampleTail tail, WidePlan plan) {
    sample_wide_body<2, kTen, kOneWide, false, NoNext, kLightCopyWaves>(sum, uniforms, depth, groups, batch, capacity, seed, calls,
                                                                       tail, plan, NoNext{});
}

// Sample plus, in the same launch, one wide field gathered at the slot each sampled row names (see kNext above).
template <int kInF, bool kTen, bool kOneWide>
__global__ __launch_bounds__(kWideWG) void k_per_sample_next(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                             int depth, uint32_t groups, int batch, uint32_t capacity,
                                                             uint64_t seed, uint64_t calls, SampleTail tail, WidePlan plan,
                                                             NextPlan nx) {
    sample_wide_body<kInF, kTen, kOneWide, true>(sum, uniforms, depth, groups, batch, capacity, seed, calls, tail, plan, nx);
}

// ---------------------------------------------------------------------------
// PER sample of rows of up to a few kilobytes (a CartPole or MuJoCo transition, an Ape-X row of 521 bytes): ONE
// WAVE per sampled row instead of a workgroup of five or six - the wave walks the tree, requests its row, takes
// the importance weight while the row is on its way, and stores. No LDS, no barrier, a sixth of the waves to
// dispatch. The walk's first node group is requested before anything else; the field table (kernel arguments,
// a trip to memory of their own when a kernel starts) is read while that group is on its way. Same outputs,
// bit for bit, as k_per_sample_wide. Rows of at most kRowWaveInF * 64 wide granules (4 KB in 16-byte fields).
// ---------------------------------------------------------------------------
constexpr int kRowWaveInF = 4;
constexpr int kRowWaveWG = 256;  // four rows per workgroup

template <bool kTen>
__global__ __launch_bounds__(kRowWaveWG) void k_per_sample_rows(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                                int depth, uint32_t groups, int batch, uint32_t capacity,
                                                                uint64_t seed, uint64_t calls, int64_t nrows, SampleTail tail,
                                                                WidePlan plan) {
    const int lane = threadIdx.x & 63;
    const int64_t k = (int64_t)blockIdx.x * (kRowWaveWG / 64) + (threadIdx.x >> 6);  // output row
    if (k >= nrows) return;  // wave-uniform
    uint32_t stratum = (uint32_t)k, nth = 0;
    if (groups >> 20) {  // several batches in the launch, each stratified on its own
        nth = (uint32_t)k / (uint32_t)batch;
        stratum = (uint32_t)k - nth * (uint32_t)batch;
    }
    CopyWork<kRowWaveInF, false, 64> work;
    NarrowWork nw;
    const bool narrow = plan.narrow_items != 0;
    const int ngroups = (int)(groups & 15u);
    uint32_t node = 1;
    float picked, mass = 0.0f, total;
    if (depth >= 2) {
        uint32_t packed = (groups >> 4) & 0x7fffu;
        int g = kTen ? kGroupMaxLevels : (int)(packed & 31u);
        f32x4 r0, r1, r2, r3;
        group_request(sum, 1u, g, lane, r0, r1, r2, r3);
        total = sum[1];
        const float u_given = *(uniforms ? uniforms + k : sum + 1);
        const uint64_t calls_now = generator_calls(uniforms, calls, tail.size, tail.err);
        __builtin_amdgcn_sched_barrier(0);
        // the field table, while the first group is on its way
        work.prepare(plan, k, 0, (uint32_t)lane);
        if (narrow) nw.prepare(plan, k, (uint32_t)lane);
        const float u = uniforms ? u_given : rng_uniform(seed, calls_now + nth, (uint64_t)stratum);
        mass = (u + (float)stratum) * (total / (float)batch);  // each operation rounded once
        node = (1u << g) + group_walk(group_finish(g, lane, r0, r1, r2, r3), g, lane, mass, picked);
#pragma nounroll
        for (int i = 1; i < ngroups; ++i) {
            packed >>= 5;
            g = kTen ? kGroupMaxLevels : (int)(packed & 31u);
            group_request(sum, node, g, lane, r0, r1, r2, r3);
            __builtin_amdgcn_sched_barrier(0);
            node = (node << g) + group_walk(group_finish(g, lane, r0, r1, r2, r3), g, lane, mass, picked);
        }
    } else {
        total = sum[1];
        const float u = uniforms ? uniforms[k] : rng_uniform(seed, generator_calls(uniforms, calls, tail.size, tail.err) + nth, (uint64_t)stratum);
        work.prepare(plan, k, 0, (uint32_t)lane);
        if (narrow) nw.prepare(plan, k, (uint32_t)lane);
        mass = (u + (float)stratum) * (total / (float)batch);
        picked = total;
        node = (1u << depth) + (depth ? group_walk(group_load_tiny(sum, 1u, depth, lane), depth, lane, mass, picked) : 0u);
    }
    const int64_t idx = (int64_t)node - ((int64_t)1 << depth);
    // the descent can end on an unfilled leaf past the last row (flagged below); the copy stays inside the storage
    const uint32_t slot = (uint32_t)(idx < (int64_t)capacity ? idx : (int64_t)capacity - 1);
    // the row: every load before the weight's arithmetic, every store after it
    uint8_t nheld[kNarrowInF];
    granule_t held[kRowWaveInF];
    if (narrow) nw.load(slot, nheld);
    if (work.live) {
#pragma unroll
        for (int j = 0; j < kRowWaveInF; ++j) held[j] = __builtin_nontemporal_load((const g16*)(work.base[j] + (uint64_t)slot * work.rb[j]));
    }
    int64_t size = tail.size;
    if (size < 0) size = counters_behind(tail.err)[kCntSize];  // device-resident counters (see Counters)
    const float fsize = (float)size;
    const float x = lane == 0 ? picked : tail.mn[1];
    float r = 0.0f;
    if (lane < 2) r = powf_det_call(x / total * fsize, -tail.beta);  // lane 0: the row's power, lane 1: the minimum's
    const float max_w = __shfl(r, 1);
    if (lane == 0) {
        tail.out_idx[k] = idx;
        tail.out_w[k] = r / max_w;
        if (!(total > 0.0f) || total > 3.0e38f) atomicOr(tail.err, MRB_DERR_TOTAL);
        if (idx >= size) atomicOr(tail.err, MRB_DERR_UNFILLED);
    }
    if (work.live) {
#pragma unroll
        for (int j = 0; j < kRowWaveInF; ++j) asm volatile("" : "+v"(held[j]));
#pragma unroll
        for (int j = 0; j < kRowWaveInF; ++j)
            if (work.live & (1u << j)) *work.dst[j] = held[j];
    }
    if (narrow) nw.store(slot, nheld, plan, (uint32_t)lane);
}

// Gather of wide rows: io_f[k] = store_f[slot_k], slot_k being `fixed_slot` (mode kFromFixedSlot, a
// single-row read), given[k] (kFromIndices) or drawn by the counter-based generator uniformly in
// [0, count) (kFromGenerator). Replaces P.BufferSample / P.BufferGetItem
// (mindspore_rl/core/uniform_replay_buffer.py:83-89,128,139) for wide rows.
constexpr int kFromIndices = 1, kFromGenerator = 2, kFromFixedSlot = 3;

template <int kInF, bool kOneWide>
__global__ __launch_bounds__(kWideWG) void k_rows_gather_wide(const int64_t* __restrict__ given, int mode,
                                                              int64_t count, int64_t fixed_slot, uint64_t seed,
                                                              uint64_t calls, int64_t* __restrict__ out_idx,
                                                              uint32_t* __restrict__ err, WidePlan plan) {
    __shared__ int64_t s_idx;
    const int64_t k = blockIdx.x;      // row
    const uint32_t part = blockIdx.y;  // which of the row's workgroups
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const bool walker = wave == 0;
    const uint32_t ctid = threadIdx.x - 64;
    CopyWork<kInF, kOneWide> work;
    NarrowWork nw;
    const bool narrow = wave == 1 + kCopyWaves && part == 0 && plan.narrow_items;
    if (walker) {
        if (lane == 0) {
            // out-of-range slots are clamped and flagged (a fixed slot was range-checked by the host
            // against the ring: it may lie above `count` after a reset)
            int64_t slot = mode == kFromFixedSlot ? fixed_slot
                           : mode == kFromIndices ? given[k]
                                                  : rng_below(seed, calls, (uint64_t)k, count);
            if (mode != kFromFixedSlot && (slot < 0 || slot >= count)) {
                if (part == 0) atomicOr(err, MRB_DERR_INDEX);
                slot = slot < 0 ? 0 : (count > 0 ? count - 1 : 0);
            }
            s_idx = slot;
            if (part == 0 && out_idx) out_idx[k] = slot;
        }
    } else {
        if (narrow) nw.prepare(plan, k, lane);
        work.prepare(plan, k, part, ctid);
    }
    __syncthreads();
    if (!walker) work.run((uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)s_idx), plan, narrow, nw, lane);
}

// Three levels of the descent from the eight nodes three levels under a node (lo: the first four, hi: the last
// four): which of them the mass falls into, what is left of the mass inside it, and its value. The sums of the
// two levels between are the single additions the tree was built with.
__device__ __forceinline__ uint32_t walk8(const float4 lo, const float4 hi, float& mass, float& picked) {
    const float a0 = lo.x + lo.y, a1 = lo.z + lo.w, a2 = hi.x + hi.y;
    const float b0 = a0 + a1;
    uint32_t p = 0;
    if (!(mass <= b0)) {
        mass -= b0;
        p = 4;
    }
    const float left1 = p ? a2 : a0;
    if (!(mass <= left1)) {
        mass -= left1;
        p += 2;
    }
    const float n0 = p == 0 ? lo.x : p == 2 ? lo.z : p == 4 ? hi.x : hi.z;
    const float n1 = p == 0 ? lo.y : p == 2 ? lo.w : p == 4 ? hi.y : hi.w;
    if (!(mass <= n0)) {
        mass -= n0;
        p += 1;
        picked = n1;
    } else {
        picked = n0;
    }
    return p;
}

// Two levels, and one, of the same descent.
__device__ __forceinline__ uint32_t walk4(const float4 v, float& mass, float& picked) {
    const float left = v.x + v.y;
    uint32_t p = 0;
    if (!(mass <= left)) {
        mass -= left;
        p = 2;
    }
    const float n0 = p ? v.z : v.x, n1 = p ? v.w : v.y;
    if (!(mass <= n0)) {
        mass -= n0;
        p += 1;
        picked = n1;
    } else {
        picked = n0;
    }
    return p;
}
__device__ __forceinline__ uint32_t walk2(const float2 pair, float& mass, float& picked) {
    if (mass <= pair.x) {
        picked = pair.x;
        return 0;
    }
    mass -= pair.x;
    picked = pair.y;
    return 1;
}

// One dependent load of the thread-per-stratum descent: the 2^g descendants of `node` g levels down (g <= 5: at most
// one cache line), the levels between rebuilt with the additions the tree was built with. Returns the node the
// mass falls into, g levels down; `mass` becomes what is left of it inside that node, `picked` the node's value.
__device__ __forceinline__ uint32_t descend_group(const float* __restrict__ sum, uint32_t node, int g, float& mass, float& picked) {
    if (g == 5) {
        const f32x4* src = reinterpret_cast<const f32x4*>(sum + ((uint64_t)node << 5));
        const f32x4 t0 = src[0], t1 = src[1], t2 = src[2], t3 = src[3], t4 = src[4], t5 = src[5], t6 = src[6], t7 = src[7];
        const f32x16 lo = __builtin_shufflevector(__builtin_shufflevector(t0, t1, 0, 1, 2, 3, 4, 5, 6, 7),
                                                  __builtin_shufflevector(t2, t3, 0, 1, 2, 3, 4, 5, 6, 7), 0, 1,
                                                  2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
        const f32x16 hi = __builtin_shufflevector(__builtin_shufflevector(t4, t5, 0, 1, 2, 3, 4, 5, 6, 7),
                                                  __builtin_shufflevector(t6, t7, 0, 1, 2, 3, 4, 5, 6, 7), 0, 1,
                                                  2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
        node = (node << 5) + walk32(lo, hi, mass, picked);
    } else if (g == 4) {
        const f32x4* src = reinterpret_cast<const f32x4*>(sum + ((uint64_t)node << 4));
        const f32x4 t0 = src[0], t1 = src[1], t2 = src[2], t3 = src[3];
        const f32x16 v = __builtin_shufflevector(__builtin_shufflevector(t0, t1, 0, 1, 2, 3, 4, 5, 6, 7),
                                                 __builtin_shufflevector(t2, t3, 0, 1, 2, 3, 4, 5, 6, 7), 0, 1,
                                                 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15);
        node = (node << 4) + walk16(v, mass, picked);
    } else if (g == 3) {
        const float4* src = reinterpret_cast<const float4*>(sum + ((uint64_t)node << 3));
        const float4 lo = src[0], hi = src[1];
        node = (node << 3) + walk8(lo, hi, mass, picked);
    } else if (g == 2) {
        const float4 v = *reinterpret_cast<const float4*>(sum + ((uint64_t)node << 2));
        const float left = v.x + v.y;
        uint32_t p = 0;
        if (!(mass <= left)) {
            mass -= left;
            p = 2;
        }
        const float n0 = p ? v.z : v.x, n1 = p ? v.w : v.y;
        if (!(mass <= n0)) {
            mass -= n0;
            p += 1;
            picked = n1;
        } else {
            picked = n0;
        }
        node = (node << 2) + p;
    } else {
        const float2 pair = *reinterpret_cast<const float2*>(sum + 2 * (uint64_t)node);
        if (mass <= pair.x) {
            node = 2 * node;
            picked = pair.x;
        } else {
            mass -= pair.x;
            node = 2 * node + 1;
            picked = pair.y;
        }
    }
    return node;
}


// ---------------------------------------------------------------------------
// PER sample, many narrow rows: one workgroup per 256 strata. The top
// `lds_levels` levels of the sum tree (nodes [1, 2 << lds_levels)) are staged
// in LDS once per workgroup, so each thread's descent reads HBM/L2 only for
// the levels below; then the workgroup gathers its 256 rows with coalesced
// writes. Same outputs, bit for bit, as k_per_sample_wide.
// ---------------------------------------------------------------------------
// sum .. calls repeat members of `a` as plain leading parameters: those are preloaded into scalar
// registers, so the staging loads go out when the wave starts instead of a round trip to the
// kernel-argument segment later.
__global__ __launch_bounds__(kLdsWG) void k_per_sample_lds(const float* __restrict__ sum, const float* __restrict__ uniforms,
                                                        const float* __restrict__ mn, int depth, int lds_levels,
                                                        int batch, float beta, uint64_t seed, uint64_t calls,
                                                        SampleArgs a, IoTable t) {
    extern __shared__ float s_top[];  // [2 << lds_levels] floats, then kWG int64 slots
    __shared__ float s_max_w;
    const uint32_t ntop = 2u << lds_levels;
    int64_t* s_slot = reinterpret_cast<int64_t*>(s_top + (ntop < 4 ? 4 : ntop));
    const int64_t k0 = (int64_t)blockIdx.x * kWG;
    const int64_t k = k0 + threadIdx.x;
    if (threadIdx.x >= kWG) {
        // The helper wave: the weights' common denominator (pmin / total * size)^-beta, once per
        // workgroup, off the strata's path (two loads and a power: as long as staging the top).
        // (the number of stored rows: the argument, or read from the device when the counters live there)
        if (threadIdx.x == kWG) s_slot[kWG] = a.size >= 0 ? a.size : counters_behind(a.err)[kCntSize];
        __syncthreads();
        if (threadIdx.x == kWG) s_max_w = powf_det(mn[1] / sum[1] * (float)s_slot[kWG], -beta);
        __syncthreads();
        return;
    }
    // the stratum's draw is requested together with the top of the tree
    float u = 0.0f;
    if (k < batch && uniforms) u = uniforms[k];
    if (ntop >= 4) {
        for (uint32_t i = threadIdx.x * 4; i < ntop; i += kWG * 4)
            *reinterpret_cast<float4*>(s_top + i) = *reinterpret_cast<const float4*>(sum + i);
    } else if (threadIdx.x < ntop) {
        s_top[threadIdx.x] = sum[threadIdx.x];
    }
    __syncthreads();
    constexpr int kOwn = 4;  // leading fields whose row is one granule: every thread copies its own stratum's
    AnyGranule own[kOwn];
    float weight = 0.0f;
    if (k < batch) {
        const float total = s_top[1];
        if (!uniforms) u = rng_uniform(seed, generator_calls(uniforms, calls, a.size, a.err), (uint64_t)k);
        float mass = (u + (float)k) * (total / (float)batch);  // each operation rounded once
        uint32_t node = 1;
        int d = 0;
        // through the staged levels three at a time: the eight descendants of `node` three levels down are 32
        // contiguous, aligned bytes of LDS - one read instead of three dependent ones -, the two levels between
        // are rebuilt with the additions the tree was built with
        for (; d + 3 <= lds_levels; d += 3) {
            const float4 lo = *reinterpret_cast<const float4*>(s_top + ((size_t)node << 3));
            const float4 hi = *reinterpret_cast<const float4*>(s_top + ((size_t)node << 3) + 4);
            float unused;
            node = (node << 3) + walk8(lo, hi, mass, unused);
        }
        for (; d < lds_levels; ++d) {
            const float left = s_top[2 * node];
            if (mass <= left) {
                node = 2 * node;
            } else {
                mass -= left;
                node = 2 * node + 1;
            }
        }
        // Below the staged levels every dependent load brings up to five levels at once: the 32 (16, 8,
        // 4, 2) descendants of `node` five (four, ... one) levels down are 128 (64, ... 8) contiguous,
        // aligned bytes - a whole cache line in the first case; the levels between are rebuilt with
        // the additions the tree was built with. The remaining levels are taken five at a time, except
        // that seven are split 4 + 3 (5 + 1 + 1 would be a load more).
        float picked = depth <= lds_levels ? s_top[node] : 0.0f;
        while (d < depth) {  // wave-uniform
            const int rest = depth - d;
            const int g = rest >= 5 ? (rest == 7 ? 4 : 5) : rest;
            node = descend_group(sum, node, g, mass, picked);
            d += g;
        }
        const int64_t idx = (int64_t)node - ((int64_t)1 << depth);
        const int64_t slot = idx < a.capacity ? idx : a.capacity - 1;
        // the row's scalar fields are requested now, before the weight's arithmetic and the barrier
#pragma unroll
        for (int f = 0; f < kOwn; ++f)
            if (f < t.nfields && t.units[f] == 1)
                own[f].load(as_global(t.store[f]) + (uint64_t)slot * t.stride[f], t.vec_log2[f]);
        a.out_idx[k] = idx;
        const int64_t size = s_slot[kWG];  // left there by the helper wave before the first barrier
        weight = powf_det(picked / total * (float)size, -beta);
        sample_flags(a, total, idx, size);
        s_slot[threadIdx.x] = slot;
    }
    __syncthreads();
    const uint32_t rows = (uint32_t)((batch - k0) < kWG ? (batch - k0) : kWG);
    if (k < batch) {
        a.out_w[k] = weight / s_max_w;
#pragma unroll
        for (int f = 0; f < kOwn; ++f)
            if (f < t.nfields && t.units[f] == 1)
                own[f].store(as_global(t.io[f]) + (uint64_t)k * t.row_bytes[f], t.vec_log2[f]);
    }
    // fields of several granules per row (and fields past the first kOwn): coalesced over the workgroup's rows
    for (int f = 0; f < t.nfields; ++f) {
        const uint32_t units = t.units[f];
        if (f < kOwn && units == 1) continue;
        const uint32_t vl = t.vec_log2[f];
        const uint64_t work = (uint64_t)rows * units;
        for (uint64_t w = threadIdx.x; w < work; w += kWG) {
            uint64_t r;
            uint32_t u;
            split_work(w, units, r, u);
            const uint64_t off = (uint64_t)u << vl;
            copy_granule(as_global(t.io[f]) + (uint64_t)(k0 + (int64_t)r) * t.row_bytes[f] + off,
                         as_global(t.store[f]) + (uint64_t)s_slot[r] * t.stride[f] + off, vl);
        }
    }
}

// ---------------------------------------------------------------------------
// Tree updates (PriorityReplayBufferUpdate and the tree half of
// PriorityReplayBufferPush, mindspore_rl/core/priority_replay_buffer.py:67-73,
// 78-90,108-120).
//
// The reference writes one leaf at a time and walks to the root after each.
// Here a call is two or three launches:
//   k_update_stamp   every valid entry j raises stamp[index_j] to
//                    (epoch << 32 | j) with an INTEGER max, so the stamp names
//                    the last entry of the call that targets the leaf (last
//                    write wins), marks the leaf's block dirty, and folds
//                    p_j^alpha into the running max (integer max of the float
//                    bits, order-preserving for non-negative floats).
//   k_tree_update    level-synchronous rebuild, one launch per round of <= 8
//                    levels. A wave owns a tile of 256 consecutive nodes; the
//                    lowest round first replaces the leaves named by the
//                    stamps (or, for a push, the leaves of the pushed slot
//                    range). Only dirty blocks load or store.
//   k_tree_top       one workgroup rebuilds the top (<= 12 levels).
// Every parent is written as the single rounded sum / min of its two final
// children, which is what a leaf-to-root walk after the last write leaves
// behind; recomputing a clean node reproduces its bits. No float is ever
// accumulated atomically.
// ---------------------------------------------------------------------------
constexpr int kMaxRounds = 3;

struct UpdateArgs {
    // entries
    const int64_t* indices;   // NULL: entry j targets slot (first_slot + j) mod capacity
    const float* priorities;  // NULL: the targeted leaves take the running max priority as it is
    int64_t n;
    int64_t first_slot;       // negative: (pushes mod capacity), read from the device (see Counters)
    // buffer
    int64_t capacity;
    int64_t leaves;
    int depth;
    float alpha;
    uint32_t epoch;
    unsigned long long* stamp;  // [leaves]
    float* sum;
    float* mn;
    float* powered;  // [n] priorities^alpha of this call's entries (update_priorities only)
    float* maxp;  // running max priority (device scalar)
    float* maxp_next;  // a push with priorities in progress: the largest p^alpha its leaf-level waves have seen
    uint32_t* err;
    // rebuild plan: round r starts at depth lo[r] and rebuilds g[r] levels; the top starts at top_depth
    int nrounds;
    int lo[kMaxRounds];
    int g[kMaxRounds];
    int top_depth;
    uint32_t* dirty[kMaxRounds];  // per round: one epoch word per block of 1 << g[r] nodes at depth lo[r]
    int fold_max;                // push with priorities: the top workgroup also raises the running max, 1 = from a
                                 // scan of the priorities, 2 = from maxp_next, where the leaf-level waves left it
    int inline_election;         // small update_priorities: no stamp pass, the leaf-level waves scan the entries
    // sparse updates of very large trees: the lowest sparse_g0 levels are rebuilt per entry
    // (k_tree_sparse) instead of per tile
    int sparse_g0;               // 0 = not used
    int full_top;                // a push that follows an update in the same call: the top is rebuilt over all its
                                 // tiles, not only those above the pushed slots (the update changed others)
    // device-resident counters: rows this launch - the push's last - adds to them when it is done (0: none), and
    // the workgroups of this launch that read the ring position (see counters_push_done)
    int64_t advance;
    uint32_t readers;
};

__device__ __forceinline__ bool valid_priority(float p) { return p >= 0.0f && p <= 3.0e38f; }

// Folds q into the running max priority. Atomics on one address are serialised by the memory
// system (~11 ns each), so the wave first looks at the current value: the max only grows, hence a
// q that does not exceed what is already there can never matter, and nearly every wave skips.
__device__ __forceinline__ void raise_max(float* maxp, float q) {
    if (q > *reinterpret_cast<volatile float*>(maxp)) atomicMax(reinterpret_cast<unsigned int*>(maxp), __float_as_uint(q));
}

__global__ __launch_bounds__(kWG) void k_update_stamp(UpdateArgs a) {
    const int64_t j = (int64_t)blockIdx.x * kWG + threadIdx.x;
    float q = 0.0f;
    if (j < a.n) {
        const float p = a.priorities[j];
        int64_t idx = a.indices ? a.indices[j] : 0;
        const bool idx_ok = !a.indices || (idx >= 0 && idx < a.capacity);
        if (!idx_ok) atomicOr(a.err, MRB_DERR_INDEX);
        if (!valid_priority(p)) atomicOr(a.err, MRB_DERR_PRIORITY);
        if (idx_ok && valid_priority(p)) {
            q = powf_det_call(p, a.alpha);
            if (a.indices) {
                a.powered[j] = q;
                atomicMax(&a.stamp[idx], ((unsigned long long)a.epoch << 32) | (unsigned long long)j);
                if (!a.sparse_g0 && a.nrounds) a.dirty[0][idx >> a.g[0]] = a.epoch;
            }
        }
    }
    // wave max, then one integer atomic per wave
    q = wave_max(q);
    if ((threadIdx.x & 63) == 0 && q > 0.0f) raise_max(a.maxp, q);
}

// New value of leaf `leaf`, if this call writes it.
//   indices given:  the entry named by the stamp
//   range + priorities: entry (leaf - first_slot) mod capacity; an invalid priority leaves the
//                   fresh slot at the running max, as a plain push would
//   range only:     the running max priority
__device__ __forceinline__ bool leaf_value(const UpdateArgs& a, int64_t first_slot, int64_t leaf, float& q) {
    if (a.indices) {
        const unsigned long long st = a.stamp[leaf];
        if ((uint32_t)(st >> 32) != a.epoch) return false;
        q = a.powered[(uint32_t)st];  // p^alpha of the winning entry, computed by k_update_stamp with full waves
        return true;
    }
    if (leaf >= a.capacity) return false;
    int64_t j = leaf - first_slot;
    if (j < 0) j += a.capacity;
    if (j >= a.n) return false;
    if (a.priorities) {
        const float p = a.priorities[j];
        const bool ok = valid_priority(p);
        q = ok ? powf_det_call(p, a.alpha) : *a.maxp;
        if (a.fold_max == 2 && !ok) atomicOr(a.err, MRB_DERR_PRIORITY);
    } else {
        q = *a.maxp;
    }
    return true;
}

// Does the pushed slot range [first_slot, first_slot + n) mod capacity meet leaves [lo, hi)?
__device__ __forceinline__ bool range_meets(const UpdateArgs& a, int64_t first_slot, int64_t lo, int64_t hi) {
    const int64_t end = first_slot + a.n;
    if (lo < (end < a.capacity ? end : a.capacity) && hi > first_slot) return true;
    return end > a.capacity && lo < end - a.capacity;
}

// One wave rebuilds `g` levels above a tile of up to 256 consecutive nodes at depth `lo`.
//   tile       index of the tile within the level
//   sparse     skip clean blocks (rounds; g >= 2 there, so a lane's four nodes share a block):
//              a block is dirty if its word in dirty_in carries this call's epoch or, at the
//              leaf level of a push (dirty_in NULL), if it meets the pushed slot range
//   dirty_out  next round's words, marked for every block rebuilt here (may be NULL)
//   win        this wave's 256 eight-byte words of LDS, used at the leaf level of a small update
//              (a.inline_election): the wave scans the call's entries itself, the last entry
//              aimed at each of its leaves wins through an LDS integer max (last write wins),
//              and the blocks holding a winner are the dirty ones
// Lanes of clean blocks neither load nor store; the shuffles of a dirty block only mix
// lanes of that block.
// The g levels above a tile whose nodes (four per lane, vs / vm) are final: parents by in-lane
// operations and wave shuffles, stored by the lanes of dirty blocks (`active`). `first`: heap index
// of the tile's first node.
// The LDS word a small update's entry bids for its leaf with: the entry's position in the call (plus one, so
// that zero means no bid) above its priority's bits. An integer max over the bids elects the last entry aimed
// at the leaf, and the winner's priority comes back with it (no second trip to the call's arrays).
__device__ __forceinline__ unsigned long long election_key(int64_t j, float p) {
    return ((unsigned long long)(j + 1) << 32) | (unsigned long long)__float_as_uint(p);
}
__device__ __forceinline__ float elected_priority(unsigned long long key) { return __uint_as_float((uint32_t)key); }

// One butterfly step of tile_parents: level 3 + S above the tile, one node per 2^(S+1) lanes.
template <int S>
__device__ __forceinline__ void parents_step(const UpdateArgs& a, int g, uint32_t first, uint32_t lane, bool active,
                                             float& cs, float& cm) {
    cs = cs + butterfly_peer<S>(cs);
    cm = fminf(cm, butterfly_peer<S>(cm));
    if (active && g >= 3 + S && (lane & ((2u << S) - 1)) == 0) {
        a.sum[(first >> (3 + S)) + (lane >> (S + 1))] = cs;
        a.mn[(first >> (3 + S)) + (lane >> (S + 1))] = cm;
    }
}

// root_s / root_m (optional): the node eight levels above a full tile, as computed here (what is stored when g >= 8).
__device__ __forceinline__ void tile_parents(const UpdateArgs& a, int g, uint32_t first, uint32_t lane, bool active,
                                             const float4& vs, const float4& vm, float* root_s = nullptr,
                                             float* root_m = nullptr) {
    // one level up: two nodes per lane; two levels up: one node per lane
    const float s0 = vs.x + vs.y, s1 = vs.z + vs.w;
    const float m0 = fminf(vm.x, vm.y), m1 = fminf(vm.z, vm.w);
    float cs = s0 + s1, cm = fminf(m0, m1);
    if (active && g >= 1) {
        *reinterpret_cast<float2*>(a.sum + (first >> 1) + 2 * lane) = make_float2(s0, s1);
        *reinterpret_cast<float2*>(a.mn + (first >> 1) + 2 * lane) = make_float2(m0, m1);
    }
    if (active && g >= 2) {
        a.sum[(first >> 2) + lane] = cs;
        a.mn[(first >> 2) + lane] = cm;
    }
    // three to six levels up: 32, 16, 8, 4 nodes per full tile, a butterfly inside each row of 16 lanes
    parents_step<0>(a, g, first, lane, active, cs, cm);
    parents_step<1>(a, g, first, lane, active, cs, cm);
    parents_step<2>(a, g, first, lane, active, cs, cm);
    parents_step<3>(a, g, first, lane, active, cs, cm);
    // seven and eight levels up: the four rows' values, read as scalars (left + right as everywhere)
    const float s_lo = lane_value(cs, 0) + lane_value(cs, 16), s_hi = lane_value(cs, 32) + lane_value(cs, 48);
    const float m_lo = fminf(lane_value(cm, 0), lane_value(cm, 16)), m_hi = fminf(lane_value(cm, 32), lane_value(cm, 48));
    if (active && g >= 7 && (lane & 31) == 0) {
        a.sum[(first >> 7) + (lane >> 5)] = lane < 32 ? s_lo : s_hi;
        a.mn[(first >> 7) + (lane >> 5)] = lane < 32 ? m_lo : m_hi;
    }
    if (active && g >= 8 && lane == 0) {
        a.sum[first >> 8] = s_lo + s_hi;
        a.mn[first >> 8] = fminf(m_lo, m_hi);
    }
    if (root_s) *root_s = s_lo + s_hi;
    if (root_m) *root_m = fminf(m_lo, m_hi);
}

// root_s / root_m / rebuilt (optional, full tiles with g = 8): the tile's root as stored, and whether the tile
// was rebuilt at all (its one block was dirty).
__device__ __forceinline__ void tile_round(const UpdateArgs& a, int lo, int g, uint32_t tile, bool sparse,
                                           const uint32_t* __restrict__ dirty_in, uint32_t* __restrict__ dirty_out,
                                           int g_next, uint32_t lane, unsigned long long* win = nullptr,
                                           float* root_s = nullptr, float* root_m = nullptr, bool* rebuilt = nullptr) {
    const uint32_t level_nodes = 1u << lo;
    const bool leaf_level = lo == a.depth;
    // where a push's slots start (a.first_slot, or read from the device)
    const int64_t first_slot =
        !leaf_level || a.indices ? 0 : a.first_slot >= 0 ? a.first_slot : ring_position(counters_behind(a.err), a.capacity);
    if (level_nodes < 4) {
        // one or two nodes: scalar, lane 0
        if (lane == 0) {
            float s0 = a.sum[level_nodes], m0 = a.mn[level_nodes], q;
            if (leaf_level && leaf_value(a, first_slot, 0, q)) {
                s0 = m0 = q;
                a.sum[level_nodes] = q;
                a.mn[level_nodes] = q;
            }
            if (level_nodes == 2) {
                float s1 = a.sum[3], m1 = a.mn[3];
                if (leaf_level && leaf_value(a, first_slot, 1, q)) {
                    s1 = m1 = q;
                    a.sum[3] = q;
                    a.mn[3] = q;
                }
                if (g >= 1) {
                    a.sum[1] = s0 + s1;
                    a.mn[1] = fminf(m0, m1);
                }
            }
        }
        return;
    }
    const uint32_t tile_nodes = level_nodes < (uint32_t)kBlockNodes ? level_nodes : (uint32_t)kBlockNodes;
    const uint32_t off = tile * kBlockNodes + 4 * lane;  // this lane's first node within the level
    const uint32_t first = level_nodes + tile * kBlockNodes;  // heap index of the tile's first node
    bool active = 4 * lane < tile_nodes;
    const bool elect = leaf_level && a.inline_election && win != nullptr;
    unsigned long long w0 = 0, w1 = 0, w2 = 0, w3 = 0;  // winning entry of each of this lane's leaves (election_key)
    if (elect) {
        win[4 * lane + 0] = 0;
        win[4 * lane + 1] = 0;
        win[4 * lane + 2] = 0;
        win[4 * lane + 3] = 0;
        __builtin_amdgcn_wave_barrier();
        // four entries per lane and trip: their loads go out together, then the election
        for (int64_t base = 0; base < a.n; base += 64 * 4) {
            int64_t idx[4];
            float pr[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int64_t j = base + 64 * q + lane;
                idx[q] = j < a.n ? a.indices[j] : -1;
                pr[q] = j < a.n ? a.priorities[j] : -1.0f;
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (idx[q] >= 0 && idx[q] < a.capacity && valid_priority(pr[q]) &&
                    (uint32_t)((uint64_t)idx[q] / kBlockNodes) == tile)
                    atomicMax(&win[idx[q] % kBlockNodes], election_key(base + 64 * q + lane, pr[q]));
            }
        }
        __threadfence_block();  // LDS operations of a wave complete in order; this also stops the compiler
        __builtin_amdgcn_wave_barrier();
        w0 = win[4 * lane + 0];
        w1 = win[4 * lane + 1];
        w2 = win[4 * lane + 2];
        w3 = win[4 * lane + 3];
        const unsigned long long hit = __ballot((w0 | w1 | w2 | w3) != 0);
        const uint32_t lanes_per_block = g >= 8 ? 64u : (1u << g) / 4u;
        const unsigned long long block_lanes =
            lanes_per_block >= 64 ? ~0ull : ((1ull << lanes_per_block) - 1) << (lane & ~(lanes_per_block - 1));
        active = active && (hit & block_lanes) != 0;
    } else if (active && sparse) {
        if (dirty_in) {
            active = dirty_in[off >> g] == a.epoch;
        } else if (leaf_level && !a.indices) {
            const int64_t b0 = (int64_t)(off >> g) << g;
            active = range_meets(a, first_slot, b0, b0 + (1ll << g));
        }
    }
    float4 vs = make_float4(0.f, 0.f, 0.f, 0.f), vm = vs;
    if (active) {
        vs = *reinterpret_cast<const float4*>(a.sum + first + 4 * lane);
        vm = *reinterpret_cast<const float4*>(a.mn + first + 4 * lane);
        if (leaf_level) {
            float q;
            bool wrote = false;
            if (elect) {
                if (w0 | w1 | w2 | w3) {
                    const float4 pw = powf_det_x4(make_float4(elected_priority(w0), elected_priority(w1), elected_priority(w2),
                                                              elected_priority(w3)), a.alpha);  // the four together
                    if (w0) vs.x = vm.x = pw.x;
                    if (w1) vs.y = vm.y = pw.y;
                    if (w2) vs.z = vm.z = pw.z;
                    if (w3) vs.w = vm.w = pw.w;
                    wrote = true;
                }
            } else if (!a.indices && a.priorities) {
                // a push with priorities: the lane's four priorities are requested together, then raised to
                // alpha one after the other (asked for one by one, each power would wait for its own load)
                float pv[4];
                bool in[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    int64_t j = (int64_t)off + c - first_slot;
                    if (j < 0) j += a.capacity;
                    in[c] = (int64_t)off + c < a.capacity && j < a.n;
                    pv[c] = in[c] ? a.priorities[j] : 0.0f;
                }
                if (in[0] || in[1] || in[2] || in[3]) {
                    const float4 pw = powf_det_x4(make_float4(pv[0], pv[1], pv[2], pv[3]), a.alpha);  // the four together
                    const float qv[4] = {pw.x, pw.y, pw.z, pw.w};
                    float* const vsp[4] = {&vs.x, &vs.y, &vs.z, &vs.w};
                    float* const vmp[4] = {&vm.x, &vm.y, &vm.z, &vm.w};
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if (in[c]) {
                            const bool ok = valid_priority(pv[c]);
                            *vsp[c] = *vmp[c] = ok ? qv[c] : *a.maxp;  // invalid: the fresh slot stays at the running max
                            if (a.fold_max == 2 && !ok) atomicOr(a.err, MRB_DERR_PRIORITY);
                            wrote = true;
                        }
                    }
                }
            } else {
                if (leaf_value(a, first_slot, off + 0, q)) { vs.x = vm.x = q; wrote = true; }
                if (leaf_value(a, first_slot, off + 1, q)) { vs.y = vm.y = q; wrote = true; }
                if (leaf_value(a, first_slot, off + 2, q)) { vs.z = vm.z = q; wrote = true; }
                if (leaf_value(a, first_slot, off + 3, q)) { vs.w = vm.w = q; wrote = true; }
            }
            if (wrote) {
                *reinterpret_cast<float4*>(a.sum + first + 4 * lane) = vs;
                *reinterpret_cast<float4*>(a.mn + first + 4 * lane) = vm;
            }
        }
        if (dirty_out && ((off & ((1u << g) - 1)) == 0)) dirty_out[(off >> g) >> g_next] = a.epoch;
    }
    if (leaf_level && a.fold_max == 2) {
        // the largest leaf of the tile bounds every p^alpha written here from above, and is itself a p^alpha or
        // a value no larger than the running max: folding it in raises the running max to exactly what a pass
        // over the call's priorities would
        float q = active ? fmaxf(fmaxf(vs.x, vs.y), fmaxf(vs.z, vs.w)) : 0.0f;
        q = wave_max(q);
        if (lane == 0 && q > 0.0f) raise_max(a.maxp_next, q);
    }
    tile_parents(a, g, first, lane, active, vs, vm, root_s, root_m);
    if (rebuilt) *rebuilt = __any(active);
}

// ---------------------------------------------------------------------------
// Sparse lowest round for very large trees (e.g. 2^24 leaves, 65,536 entries): scanning
// every 256-leaf tile costs more in wave launches than the update itself, so here the
// ENTRIES drive the work. A group of L = 2^(g0-2) lanes (g0 = 4..6) takes one entry; if
// that entry owns its block of 2^g0 leaves (it holds the largest of the block's stamps), the
// group loads the block, replaces the leaves the stamps name, rebuilds the g0 levels
// above with the same pairwise operations as tile_round and marks the next round's block.
// ---------------------------------------------------------------------------
// One butterfly step of k_tree_sparse inside an entry's group of lanes: level 3 + S above its block.
template <int S>
__device__ __forceinline__ void sparse_step(const UpdateArgs& a, int g0, uint64_t first, uint32_t sub, bool active,
                                            float& cs, float& cm) {
    if (S < g0 - 2) {  // wave-uniform
        cs = cs + butterfly_peer<S>(cs);
        cm = fminf(cm, butterfly_peer<S>(cm));
        if (active && (sub & ((2u << S) - 1)) == 0) {
            a.sum[(first >> (3 + S)) + (sub >> (S + 1))] = cs;
            a.mn[(first >> (3 + S)) + (sub >> (S + 1))] = cm;
        }
    }
}

__global__ __launch_bounds__(kWG) void k_tree_sparse(UpdateArgs a) {
    const int g0 = a.sparse_g0;
    const uint32_t group = 1u << (g0 - 2);
    const uint64_t tid = (uint64_t)blockIdx.x * kWG + threadIdx.x;
    const int64_t j = (int64_t)(tid >> (g0 - 2));
    const uint32_t sub = (uint32_t)tid & (group - 1);
    bool active = j < a.n;
    int64_t idx = 0;
    if (active) {
        idx = a.indices[j];
        active = idx >= 0 && idx < a.capacity && valid_priority(a.priorities[j]);
    }
    const uint64_t block = (uint64_t)idx >> g0;
    const uint64_t first = (uint64_t)a.leaves + (block << g0);  // heap index of the block's first leaf
    // The block's owner is the entry with the largest stamp of this call among its leaves: every
    // group aimed at the block reads the same 2^g0 stamps and only the owner's group goes on.
    unsigned long long top = 0;
    if (active) {
        const unsigned long long* st = a.stamp + (block << g0) + 4 * sub;
        const unsigned long long s0 = st[0], s1 = st[1], s2 = st[2], s3 = st[3];
        top = s0 > s1 ? s0 : s1;
        top = top > s2 ? top : s2;
        top = top > s3 ? top : s3;
    }
    for (uint32_t m = 1; m < group; m <<= 1) {
        const unsigned long long o = __shfl_xor(top, (int)m);
        top = top > o ? top : o;
    }
    active = active && top == (((unsigned long long)a.epoch << 32) | (unsigned long long)j);
    float4 vs = make_float4(0.f, 0.f, 0.f, 0.f), vm = vs;
    if (active) {
        vs = *reinterpret_cast<const float4*>(a.sum + first + 4 * sub);
        vm = *reinterpret_cast<const float4*>(a.mn + first + 4 * sub);
        const int64_t leaf0 = (int64_t)((block << g0) + 4 * sub);
        float q;
        bool wrote = false;
        if (leaf_value(a, 0, leaf0 + 0, q)) { vs.x = vm.x = q; wrote = true; }
        if (leaf_value(a, 0, leaf0 + 1, q)) { vs.y = vm.y = q; wrote = true; }
        if (leaf_value(a, 0, leaf0 + 2, q)) { vs.z = vm.z = q; wrote = true; }
        if (leaf_value(a, 0, leaf0 + 3, q)) { vs.w = vm.w = q; wrote = true; }
        if (wrote) {
            *reinterpret_cast<float4*>(a.sum + first + 4 * sub) = vs;
            *reinterpret_cast<float4*>(a.mn + first + 4 * sub) = vm;
        }
        if (sub == 0 && a.nrounds) a.dirty[0][block >> a.g[0]] = a.epoch;
    }
    const float s0 = vs.x + vs.y, s1 = vs.z + vs.w;
    const float m0 = fminf(vm.x, vm.y), m1 = fminf(vm.z, vm.w);
    float cs = s0 + s1, cm = fminf(m0, m1);
    if (active) {
        *reinterpret_cast<float2*>(a.sum + (first >> 1) + 2 * sub) = make_float2(s0, s1);
        *reinterpret_cast<float2*>(a.mn + (first >> 1) + 2 * sub) = make_float2(m0, m1);
        a.sum[(first >> 2) + sub] = cs;
        a.mn[(first >> 2) + sub] = cm;
    }
    sparse_step<0>(a, g0, first, sub, active, cs, cm);
    sparse_step<1>(a, g0, first, sub, active, cs, cm);
    sparse_step<2>(a, g0, first, sub, active, cs, cm);
    sparse_step<3>(a, g0, first, sub, active, cs, cm);
}

// Small update on a tree whose leaves the top workgroup itself rebuilds (no stamp pass, no wave per entry):
// what k_update_stamp does besides electing — flag invalid entries and fold every valid p^alpha into the
// running max — is shared out among the waves, 64 entries at a time. (Where a wave per entry runs,
// entry_tile does this for its own entry.)
__device__ __forceinline__ void entry_duty(const UpdateArgs& a, uint32_t wave_id, uint32_t nwaves, uint32_t lane) {
    for (int64_t base = (int64_t)wave_id * 64; base < a.n; base += (int64_t)nwaves * 64) {
        const int64_t j = base + lane;
        float q = 0.0f;
        if (j < a.n) {
            const int64_t idx = a.indices[j];
            const float p = a.priorities[j];
            const bool idx_ok = idx >= 0 && idx < a.capacity;
            if (!idx_ok) atomicOr(a.err, MRB_DERR_INDEX);
            if (!valid_priority(p)) atomicOr(a.err, MRB_DERR_PRIORITY);
            if (idx_ok && valid_priority(p)) q = powf_det_call(p, a.alpha);
        }
        q = wave_max(q);
        if (lane == 0 && q > 0.0f) raise_max(a.maxp, q);
    }
}

// A push with priorities raises the running max to the largest p^alpha of the call, after the tree
// work: the leaves read the running max as it was before the call (a fresh slot with an invalid
// priority takes it), so every wave of the top workgroup passes the barrier before any raises it.
__device__ __forceinline__ void fold_push_max(const UpdateArgs& a) {
    __syncthreads();
    if (a.fold_max == 2) {
        // collected by the leaf-level waves, in this launch or the ones before it
        if (threadIdx.x == 0) {
            // taken and set back to zero in one atomic, where the waves' atomic maxima were performed
            const float q = __uint_as_float(atomicExch(reinterpret_cast<unsigned int*>(a.maxp_next), 0u));
            if (q > 0.0f) raise_max(a.maxp, q);
        }
        return;
    }
    float q = 0.0f;
    for (int64_t j = threadIdx.x; j < a.n; j += blockDim.x) {
        const float p = a.priorities[j];
        if (valid_priority(p)) {
            q = fmaxf(q, powf_det_call(p, a.alpha));
        } else {
            atomicOr(a.err, MRB_DERR_PRIORITY);
        }
    }
    q = wave_max(q);
    if ((threadIdx.x & 63) == 0 && q > 0.0f) raise_max(a.maxp, q);
}

// A small update, driven by its entries: the 256-leaf tile that entry j falls into is rebuilt with every entry
// of the call that falls into it (the last one aimed at a leaf wins, elected by an LDS integer max over a scan
// of the call's entries), and the g levels above it. Entries that share a tile have the same values written
// to the same nodes. The pieces below are put together twice: entry_tile (one wave does everything) and
// entry_pair (two waves share an entry: one takes the power and the tile, the other the election).
constexpr int kScanPer = 8;  // entries per lane and trip of the scan: a call of up to 512 entries is one trip,
                             // all of its loads requested before anything waits

// Requests the first trip's entries.
__device__ __forceinline__ void scan_request(const UpdateArgs& a, uint32_t lane, int64_t (&idx)[kScanPer], float (&pr)[kScanPer]) {
#pragma unroll
    for (int q = 0; q < kScanPer; ++q) {
        const int64_t e = 64 * q + lane;
        idx[q] = e < a.n ? a.indices[e] : -1;
        pr[q] = e < a.n ? a.priorities[e] : -1.0f;
    }
}

__device__ __forceinline__ void clear_bids(unsigned long long* win, uint32_t lane) {
    win[4 * lane + 0] = 0;
    win[4 * lane + 1] = 0;
    win[4 * lane + 2] = 0;
    win[4 * lane + 3] = 0;
}

// Every valid entry of the call that falls into `tile` bids for its leaf (idx / pr hold the first trip).
__device__ __forceinline__ void scan_bids(const UpdateArgs& a, uint32_t tile, uint32_t lane, unsigned long long* win,
                                          int64_t (&idx)[kScanPer], float (&pr)[kScanPer]) {
    for (int64_t base = 0; base < a.n; base += 64 * kScanPer) {
        if (base > 0) {
#pragma unroll
            for (int q = 0; q < kScanPer; ++q) {
                const int64_t e = base + 64 * q + lane;
                idx[q] = e < a.n ? a.indices[e] : -1;
                pr[q] = e < a.n ? a.priorities[e] : -1.0f;
            }
        }
#pragma unroll
        for (int q = 0; q < kScanPer; ++q) {
            if (base + 64 * q >= a.n) break;  // wave-uniform: no entries left
            if (idx[q] >= 0 && idx[q] < a.capacity && valid_priority(pr[q]) &&
                (uint32_t)((uint64_t)idx[q] / kBlockNodes) == tile)
                atomicMax(&win[idx[q] % kBlockNodes], election_key(base + 64 * q + lane, pr[q]));  // the last entry wins
        }
    }
}

// What k_update_stamp does for an entry besides electing: flags it if it is invalid. Returns whether it is valid.
__device__ __forceinline__ bool entry_valid(const UpdateArgs& a, int64_t idx_j, float p_j, uint32_t lane, bool flag) {
    const bool idx_ok = idx_j >= 0 && idx_j < a.capacity, p_ok = valid_priority(p_j);
    if (flag && lane == 0 && !idx_ok) atomicOr(a.err, MRB_DERR_INDEX);
    if (flag && lane == 0 && !p_ok) atomicOr(a.err, MRB_DERR_PRIORITY);
    return idx_ok && p_ok;
}

// After the election: the tile (vs / vm as memory held it) takes the winners' powers, is stored, and its g
// levels of parents with it. q_j: p^alpha of entry j, the power nearly every leaf written here gets; the other
// entries that won a leaf of the tile (few, if any) take theirs together, one per lane and trip.
// dirty_out: the next round's words, marked for every block rebuilt here (NULL when the top comes next).
__device__ __forceinline__ void entry_finish(const UpdateArgs& a, int g, uint32_t j, uint32_t tile, uint32_t lane,
                                             const unsigned long long* win, float4 vs, float4 vm, float q_j,
                                             uint32_t* __restrict__ dirty_out, int g_next) {
    const uint32_t first = (1u << a.depth) + tile * kBlockNodes;
    const unsigned long long w0 = win[4 * lane + 0], w1 = win[4 * lane + 1], w2 = win[4 * lane + 2], w3 = win[4 * lane + 3];
    const unsigned long long hit = __ballot((w0 | w1 | w2 | w3) != 0);
    const uint32_t lanes_per_block = g >= 8 ? 64u : (1u << g) / 4u;
    const unsigned long long block_lanes =
        lanes_per_block >= 64 ? ~0ull : ((1ull << lanes_per_block) - 1) << (lane & ~(lanes_per_block - 1));
    const bool active = (hit & block_lanes) != 0;  // this lane's block of 2^g leaves holds a winner
    const unsigned long long own = (unsigned long long)(j + 1) << 32;
    uint32_t pending = 0;
    if (w0) { if ((w0 >> 32 << 32) == own) vs.x = vm.x = q_j; else pending |= 1u; }
    if (w1) { if ((w1 >> 32 << 32) == own) vs.y = vm.y = q_j; else pending |= 2u; }
    if (w2) { if ((w2 >> 32 << 32) == own) vs.z = vm.z = q_j; else pending |= 4u; }
    if (w3) { if ((w3 >> 32 << 32) == own) vs.w = vm.w = q_j; else pending |= 8u; }
    while (__any(pending != 0)) {
        if (pending) {
            const int c = __ffs(pending) - 1;
            const unsigned long long w = c == 0 ? w0 : c == 1 ? w1 : c == 2 ? w2 : w3;
            const float q = powf_det_call(elected_priority(w), a.alpha);
            if (c == 0) vs.x = vm.x = q;
            if (c == 1) vs.y = vm.y = q;
            if (c == 2) vs.z = vm.z = q;
            if (c == 3) vs.w = vm.w = q;
            pending &= pending - 1;
        }
    }
    if (w0 | w1 | w2 | w3) {
        *reinterpret_cast<float4*>(a.sum + first + 4 * lane) = vs;
        *reinterpret_cast<float4*>(a.mn + first + 4 * lane) = vm;
    }
    const uint32_t off = tile * kBlockNodes + 4 * lane;  // this lane's first leaf
    if (active && dirty_out && (off & ((1u << g) - 1)) == 0) dirty_out[(off >> g) >> g_next] = a.epoch;
    tile_parents(a, g, first, lane, active, vs, vm);
}

// One wave per entry. The loads are kept apart from what they do not depend on: the entry, the first entries
// of the scan and then the tile are requested before anything is computed.
__device__ __forceinline__ void entry_tile(const UpdateArgs& a, int g, uint32_t j, uint32_t lane, unsigned long long* win,
                                           uint32_t* __restrict__ dirty_out, int g_next) {
    int64_t idx[kScanPer];
    float pr[kScanPer];
    const int64_t idx_j = a.indices[j];
    const float p_j = a.priorities[j];
    scan_request(a, lane, idx, pr);
    clear_bids(win, lane);
    if (!entry_valid(a, idx_j, p_j, lane, true)) return;  // wave-uniform: an entry that is skipped
    const uint32_t tile = (uint32_t)((uint64_t)idx_j / kBlockNodes);
    const uint32_t first = (1u << a.depth) + tile * kBlockNodes;
    const float4 vs = *reinterpret_cast<const float4*>(a.sum + first + 4 * lane);
    const float4 vm = *reinterpret_cast<const float4*>(a.mn + first + 4 * lane);
    // The entry's p^alpha, folded into the running max as k_update_stamp would. The power is taken here, inlined,
    // while the tile and the scan's entries are on their way (a call would wait for every load in flight first):
    // it is nearly always the value this wave's own leaf gets, and it costs as much as the tile's trip to memory.
    const float q_j = powf_det(p_j, a.alpha);
    if (lane == 0 && q_j > 0.0f) raise_max(a.maxp, q_j);
    __builtin_amdgcn_wave_barrier();
    scan_bids(a, tile, lane, win, idx, pr);
    __threadfence_block();  // LDS operations of a wave complete in order; this also stops the compiler
    __builtin_amdgcn_wave_barrier();
    entry_finish(a, g, j, tile, lane, win, vs, vm, q_j, dirty_out, g_next);
}

// Calls of more entries than this give each entry two waves (entry_pair): the scan of a short call is too short
// to be worth a second wave and a barrier (64 entries: no gain on the call, 0.5 us lost in a loop of calls).
constexpr int64_t kPairedAbove = 128;

// Two waves per entry (`role` 0 and 1, in one workgroup, `win` shared by the two): the power - some 110
// dependent double-precision operations - and the election are each a wave's worth of instructions in a row;
// side by side they take the time of the longer one. Every wave of the workgroup reaches the one barrier.
__device__ __forceinline__ void entry_pair(const UpdateArgs& a, int g, uint32_t j, uint32_t role, uint32_t lane,
                                           unsigned long long* win, uint32_t* __restrict__ dirty_out, int g_next) {
    const bool have = (int64_t)j < a.n;  // wave-uniform
    const int64_t idx_j = have ? a.indices[j] : -1;
    const float p_j = have ? a.priorities[j] : -1.0f;
    if (role == 1) {
        // the election
        int64_t idx[kScanPer];
        float pr[kScanPer];
        if (have) scan_request(a, lane, idx, pr);
        clear_bids(win, lane);
        if (have && entry_valid(a, idx_j, p_j, lane, false))
            scan_bids(a, (uint32_t)((uint64_t)idx_j / kBlockNodes), lane, win, idx, pr);
        lds_barrier();
        return;
    }
    // the tile and the power
    const bool valid = have && entry_valid(a, idx_j, p_j, lane, true);
    const uint32_t tile = valid ? (uint32_t)((uint64_t)idx_j / kBlockNodes) : 0u;
    const uint32_t first = (1u << a.depth) + tile * kBlockNodes;
    float4 vs = make_float4(0.f, 0.f, 0.f, 0.f), vm = vs;
    float q_j = 0.0f;
    if (valid) {
        vs = *reinterpret_cast<const float4*>(a.sum + first + 4 * lane);
        vm = *reinterpret_cast<const float4*>(a.mn + first + 4 * lane);
        q_j = powf_det(p_j, a.alpha);
        if (lane == 0 && q_j > 0.0f) raise_max(a.maxp, q_j);
    }
    lds_barrier();
    if (valid) entry_finish(a, g, j, tile, lane, win, vs, vm, q_j, dirty_out, g_next);
}

// Rebuilds everything above depth `top` (<= 16) with one workgroup: first up to 8 levels over
// the tiles of that depth (shared out among the waves), then the rest in one tile. When `top`
// is the leaf level, clean tiles are skipped like in a round. `win`: 256 eight-byte words of LDS per wave
// (see tile_round).
__device__ __forceinline__ void top_rebuild(const UpdateArgs& a, int top, unsigned long long* win) {
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int g1 = top < kRoundLevels ? top : kRoundLevels;
    const uint32_t tiles = (1u << top) <= (uint32_t)kBlockNodes ? 1u : (1u << top) / kBlockNodes;
    if (a.inline_election && top == a.depth) entry_duty(a, wave, nwaves, lane);
    // A push that does not wrap changed the nodes above one run of slots only: above the leaf level, the
    // tiles outside that run hold what they held, and the waves they would occupy stay out of the way.
    uint32_t t_lo = 0, t_hi = tiles - 1;
    if (!a.indices && !a.full_top && top != a.depth) {
        // (the slots' start: an argument, or read from the device - the leaf tiles' waves have just read it)
        const int64_t first_slot = a.first_slot >= 0 ? a.first_slot : ring_position(counters_behind(a.err), a.capacity);
        if (first_slot + a.n <= a.capacity) {
            t_lo = (uint32_t)(first_slot >> (a.depth - top)) / kBlockNodes;
            t_hi = (uint32_t)((first_slot + a.n - 1) >> (a.depth - top)) / kBlockNodes;
        }
    }
    if (top != a.depth && g1 == kRoundLevels) {
        // full tiles above the leaf level: nothing to elect, no clean blocks - the nodes and their eight levels
        // of parents, without tile_round's cases (sixteen waves share this compute unit's issue slots)
        for (uint32_t t = t_lo + wave; t <= t_hi; t += nwaves) {
            const uint32_t first = (1u << top) + t * kBlockNodes;
            const float4 vs = *reinterpret_cast<const float4*>(a.sum + first + 4 * lane);
            const float4 vm = *reinterpret_cast<const float4*>(a.mn + first + 4 * lane);
            tile_parents(a, kRoundLevels, first, lane, true, vs, vm);
        }
    } else {
        for (uint32_t t = t_lo + wave; t <= t_hi; t += nwaves)
            tile_round(a, top, g1, t, top == a.depth && g1 >= 2, nullptr, nullptr, 0, lane, win + wave * kBlockNodes);
    }
    if (top > g1) {
        __threadfence_block();  // the tiles' parents, written by other waves of this workgroup, are read below
        __syncthreads();
        if (wave == 0) tile_round(a, top - g1, top - g1, 0, false, nullptr, nullptr, 0, lane);
    }
}

// One wave per tile of round `round` (>= 0). A push lets its row copy ride along in the same
// launch (the copy and the tree work touch different memory): workgroups past the tiles do it.
// `tile_base`: the launch covers tiles tile_base, tile_base + 1, ... only (a push knows which leaf
// tiles its slot range meets).
// The leading plain parameters repeat members of `a_in` (plan: round | lo[round] << 8 | g[round] << 16): they are
// preloaded into scalar registers, so an entry-driven round requests its entries when a wave starts and the tiles
// when the entries have arrived, not a trip to the kernel-argument segment later.
__global__ __launch_bounds__(kWG) void k_tree_update(const int64_t* __restrict__ lead_indices,
                                                     const float* __restrict__ lead_priorities, float* lead_sum, float* lead_mn,
                                                     int64_t lead_n, int64_t lead_capacity, int plan, float lead_alpha,
                                                     UpdateArgs a_in, uint32_t tile_base, PutArgs put) {
    __shared__ unsigned long long s_win[kWG / 64][kBlockNodes];
    const uint32_t tile_blocks = gridDim.x - put.blocks;
    if (blockIdx.x >= tile_blocks) {
        rows_put_part(put, blockIdx.x - tile_blocks, put.blocks);
        rider_ends();
    }
    UpdateArgs a = a_in;
    a.indices = lead_indices;
    a.priorities = lead_priorities;
    a.sum = lead_sum;
    a.mn = lead_mn;
    a.n = lead_n;
    a.capacity = lead_capacity;
    a.alpha = lead_alpha;
    const int round = plan & 255;
    const uint32_t lane = threadIdx.x & 63;
    const int lo = (plan >> 8) & 255, g = (plan >> 16) & 255;
    uint32_t tile = tile_base + blockIdx.x * (kWG / 64) + (threadIdx.x >> 6);
    const uint32_t ntiles = (1u << lo) / kBlockNodes;
    const bool last_round = round + 1 == a.nrounds;
    const bool elect = round == 0 && a.inline_election;
    if (elect) {
        // Small update: a wave per ENTRY, not per tile of the level. Wave j rebuilds the tile that entry j
        // falls into, with every entry of the call that falls into it; entries sharing a tile make
        // their waves write the same values to the same nodes. (4096 tiles scanned for 512 entries
        // cost three times as much as the rebuild itself.)
        uint32_t* const dirty_next = last_round ? nullptr : a_in.dirty[round + 1];
        const int g_next = last_round ? 0 : a_in.g[round + 1];
        if (a.n > kPairedAbove) {
            // two waves per entry (see entry_pair; the launch brings a workgroup per two entries)
            const uint32_t pair = threadIdx.x >> 7, role = (threadIdx.x >> 6) & 1u;
            entry_pair(a, g, blockIdx.x * (kWG / 128) + pair, role, lane, s_win[pair], dirty_next, g_next);
            return;
        }
        const uint32_t j = tile;  // tile_base is 0 here
        if ((int64_t)j >= a.n) return;
        entry_tile(a, g, j, lane, s_win[threadIdx.x >> 6], dirty_next, g_next);
        return;
    }
    if (round == 0 && !a.indices && a.first_slot < 0) {
        // a push whose slots start at a position only the device knows: the launch brings enough waves for the
        // tiles the slots can meet; they start at the tile of the first slot and wrap around the level
        const uint32_t unit = blockIdx.x * (kWG / 64) + (threadIdx.x >> 6);
        if (unit >= tile_base) return;  // tile_base carries the number of such waves here
        const uint32_t ring_tiles = (uint32_t)((a.capacity + kBlockNodes - 1) / kBlockNodes);  // the ring ends at `capacity`
        tile = ((uint32_t)(ring_position(counters_behind(a.err), a.capacity) / kBlockNodes) + unit) % ring_tiles;
    }
    if (tile >= ntiles) return;
    tile_round(a, lo, g, tile, true, (elect || (round == 0 && !a.indices)) ? nullptr : a_in.dirty[round],
               last_round ? nullptr : a_in.dirty[round + 1], last_round ? 0 : a_in.g[round + 1], lane,
               s_win[threadIdx.x >> 6]);
}

// The top of the tree (everything above a.top_depth; the whole tree, leaves included, when it has
// no rounds), one workgroup; further workgroups carry a push's row copy when the tree has no rounds.
// A separate launch rather than a continuation of the last round by its last workgroup: publishing
// the rounds' stores to that workgroup needs an agent-scope fence per workgroup, which on this
// multi-die part costs far more than a launch.
constexpr int kTopWG = 1024;
__global__ __launch_bounds__(kTopWG) void k_tree_top(UpdateArgs a, PutArgs put) {
    __shared__ unsigned long long s_win[kTopWG / 64][kBlockNodes];
    if (__builtin_expect(blockIdx.x >= 1, 0)) {  // (the tree workgroup's code comes first: it is the one the call waits for)
        rows_put_part(put, blockIdx.x - 1, put.blocks);
        counters_push_done(a.err, a.advance, a.capacity, a.readers);
        rider_ends();
    }
    // (a launch that moves the device's counters on: thread 0 takes them now, for the advance at the end)
    CounterTicket ticket{};
    if (a.advance > 0 && threadIdx.x == 0) ticket = counters_take(a.err);
    top_rebuild(a, a.top_depth, &s_win[0][0]);
    if (a.fold_max) fold_push_max(a);
    counters_push_done(a.err, a.advance, a.capacity, a.readers, &ticket);
}

// ---------------------------------------------------------------------------
// A push of few rows, or an update of at most 16 entries, on a tree with one round below the top,
// in ONE launch: the tile work fits the 16 waves of one workgroup (a wave per leaf tile of a push,
// or per entry of an update), and the same workgroup goes on to the top after a barrier. Within one
// workgroup that needs no fence: its waves share a compute unit, and the nodes the top reads were
// never in that unit's cache before they were written. (Handing the tiles of SEVERAL workgroups to a
// last one through agent-scope stores, a counter and agent-scope loads was measured too: the three
// trips through memory cost 2.9 us, more than the second launch they save.)
//   units      waves with work: entries (update) or leaf tiles from tile_base on (push), at most 16
// ---------------------------------------------------------------------------
constexpr int kFusedWG = 1024;

__global__ __launch_bounds__(kFusedWG) void k_tree_fused(UpdateArgs a, uint32_t tile_base, uint32_t units, PutArgs put) {
    __shared__ unsigned long long s_win[kFusedWG / 64][kBlockNodes];
    if (__builtin_expect(blockIdx.x >= 1, 0)) {  // (the tree workgroup's code comes first: it is the one the call waits for)
        rows_put_part(put, blockIdx.x - 1, put.blocks);
        counters_push_done(a.err, a.advance, a.capacity, a.readers);
        rider_ends();
    }
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int top = a.top_depth;
    // (a launch that moves the device's counters on: thread 0 takes them now, for the advance at the end)
    CounterTicket ticket{};
    if (a.advance > 0 && threadIdx.x == 0) ticket = counters_take(a.err);
    if (!a.inline_election && a.lo[0] == a.depth && a.g[0] == kRoundLevels && top >= kRoundLevels &&
        (1u << top) / kBlockNodes <= (uint32_t)(kFusedWG / 64)) {
        // A push: the top's tiles (one per wave) are requested BEFORE the leaf tiles are rebuilt - of all their
        // nodes only the leaf tiles' roots change, and those reach the waves that hold them through LDS - so the
        // call has two dependent trips to memory on its path (leaf tiles and top tiles together, then the last
        // tile) instead of three.
        __shared__ uint32_t s_root_tile[kFusedWG / 64];
        __shared__ float s_root_s[kFusedWG / 64], s_root_m[kFusedWG / 64];
        const uint32_t tiles = (1u << top) / kBlockNodes;
        uint32_t t_lo = 0, t_hi = tiles - 1;
        const int64_t first_slot = a.first_slot >= 0 ? a.first_slot : ring_position(counters_behind(a.err), a.capacity);
        if (!a.full_top && first_slot + a.n <= a.capacity) {
            t_lo = (uint32_t)(first_slot >> (a.depth - top)) / kBlockNodes;
            t_hi = (uint32_t)((first_slot + a.n - 1) >> (a.depth - top)) / kBlockNodes;
        }
        const bool mine = wave >= t_lo && wave <= t_hi;  // this wave rebuilds the top's tile number `wave`
        const uint32_t top_first = (1u << top) + wave * kBlockNodes;
        float4 tvs = make_float4(0.f, 0.f, 0.f, 0.f), tvm = tvs;
        if (mine) {
            tvs = *reinterpret_cast<const float4*>(a.sum + top_first + 4 * lane);
            tvm = *reinterpret_cast<const float4*>(a.mn + top_first + 4 * lane);
        }
        uint32_t leaf_tile = 0xffffffffu;
        float rs = 0.0f, rm = 0.0f;
        if (wave < units) {
            const uint32_t ring_tiles = (uint32_t)((a.capacity + kBlockNodes - 1) / kBlockNodes);  // the ring ends at `capacity`
            const uint32_t tile = a.first_slot >= 0 ? tile_base + wave
                                                    : ((uint32_t)(first_slot / kBlockNodes) + wave) % ring_tiles;
            bool rebuilt = false;
            tile_round(a, a.depth, kRoundLevels, tile, true, nullptr, nullptr, 0, lane, nullptr, &rs, &rm, &rebuilt);
            if (rebuilt) leaf_tile = tile;
        }
        if (lane == 0) {
            s_root_tile[wave] = leaf_tile;
            s_root_s[wave] = rs;
            s_root_m[wave] = rm;
        }
        lds_barrier();
        if (mine) {
            for (uint32_t u = 0; u < units; ++u) {  // uniform
                const uint32_t lt = s_root_tile[u];  // the leaf tile's number = its root's place in the top's level
                if (lt != 0xffffffffu && lt / kBlockNodes == wave && (lt % kBlockNodes) / 4 == lane) {
                    const float ps = s_root_s[u], pm = s_root_m[u];
                    switch (lt & 3u) {
                        case 0: tvs.x = ps, tvm.x = pm; break;
                        case 1: tvs.y = ps, tvm.y = pm; break;
                        case 2: tvs.z = ps, tvm.z = pm; break;
                        default: tvs.w = ps, tvm.w = pm; break;
                    }
                }
            }
            tile_parents(a, kRoundLevels, top_first, lane, true, tvs, tvm);
        }
        if (top > kRoundLevels) {
            __threadfence_block();  // the tiles' parents, written by other waves of this workgroup, are read below
            __syncthreads();
            if (wave == 0) tile_round(a, top - kRoundLevels, top - kRoundLevels, 0, false, nullptr, nullptr, 0, lane);
        }
        if (a.fold_max) fold_push_max(a);
        counters_push_done(a.err, a.advance, a.capacity, a.readers, &ticket);
        return;
    }
    if (const uint32_t unit = wave; unit < units) {
        if (a.inline_election) {
            entry_tile(a, a.g[0], unit, lane, s_win[wave], nullptr, 0);
        } else {
            // (device-resident counters: the tiles start at the first slot's tile and wrap around the level)
            const uint32_t ring_tiles = (uint32_t)((a.capacity + kBlockNodes - 1) / kBlockNodes);  // the ring ends at `capacity`
            const uint32_t tile = a.first_slot >= 0 ? tile_base + unit
                                                    : ((uint32_t)(ring_position(counters_behind(a.err), a.capacity) / kBlockNodes) + unit) % ring_tiles;
            tile_round(a, a.lo[0], a.g[0], tile, true, nullptr, nullptr, 0, lane);
        }
    }
    __threadfence_block();  // the tiles' highest nodes, written by other waves of this workgroup, are read below
    __syncthreads();
    top_rebuild(a, a.top_depth, &s_win[0][0]);
    if (a.fold_max) fold_push_max(a);
    counters_push_done(a.err, a.advance, a.capacity, a.readers, &ticket);
}

// ---------------------------------------------------------------------------
// update_priorities of at most 64 entries in ONE launch of ONE wave, along the entries' paths instead of by
// tiles: an entry changes its leaf and the `depth` nodes above it, 15 nodes of a 14-level tree where its tile
// has 511, so a single wave has time for all of it and no second launch is needed for the top.
//   1. a lane per entry; the valid ones are sorted by (leaf, position in the call) with a bitonic network. Of
//      the entries aimed at one leaf the last lane of the run - the latest entry - stays active.
//   2. every active lane requests the siblings of the nodes on its path (their addresses follow from the
//      leaf), then takes its power while they are on their way.
//   3. level by level, from the leaves up: the parent is left + right, where the other child is the lane's
//      sibling as memory holds it unless another entry of the call has changed it - then it is the value
//      that entry's lane carries, and because the active lanes stay sorted by node it can only be the next
//      active lane (for a left child) or the one before (for a right child). Of two lanes that meet in a
//      parent the left child's goes on. Every node is the single rounded sum / min of its two final
//      children, as everywhere.
// Keys are 32 bits: leaf * 64 + lane, so the tree has at most 2^25 leaves here.
// ---------------------------------------------------------------------------
constexpr int kPathEntries = 64;
constexpr int kPathMaxDepth = 25;

// The key lane ^ J holds: inside a row of 16 lanes through DPP (quad permutations, row rotations), across rows
// through the LDS crossbar.
template <uint32_t J>
__device__ __forceinline__ uint32_t xor_peer(uint32_t key, uint32_t lane) {
    if (J == 1) return (uint32_t)__builtin_amdgcn_mov_dpp((int)key, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]
    if (J == 2) return (uint32_t)__builtin_amdgcn_mov_dpp((int)key, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    if (J == 8) return (uint32_t)__builtin_amdgcn_mov_dpp((int)key, 0x128, 0xF, 0xF, true);  // row_ror:8
    if (J == 4) {
        const uint32_t up = (uint32_t)__builtin_amdgcn_mov_dpp((int)key, 0x12C, 0xF, 0xF, true);    // row_ror:12 = lane + 4
        const uint32_t down = (uint32_t)__builtin_amdgcn_mov_dpp((int)key, 0x124, 0xF, 0xF, true);  // row_ror:4 = lane - 4
        return (lane & 4u) ? down : up;
    }
    return (uint32_t)__shfl_xor((int)key, (int)J);
}

template <uint32_t K, uint32_t J>
__device__ __forceinline__ uint32_t sort_step(uint32_t key, uint32_t lane) {
    const uint32_t other = xor_peer<J>(key, lane);
    const bool take_min = ((lane & J) == 0) == ((lane & K) == 0);
    return take_min ? (key < other ? key : other) : (key > other ? key : other);
}

// Ascending bitonic sort of one key per lane over the wave.
__device__ __forceinline__ uint32_t bitonic_sort_wave(uint32_t key, uint32_t lane) {
    key = sort_step<2, 1>(key, lane);
    key = sort_step<4, 2>(key, lane);
    key = sort_step<4, 1>(key, lane);
    key = sort_step<8, 4>(key, lane);
    key = sort_step<8, 2>(key, lane);
    key = sort_step<8, 1>(key, lane);
    key = sort_step<16, 8>(key, lane);
    key = sort_step<16, 4>(key, lane);
    key = sort_step<16, 2>(key, lane);
    key = sort_step<16, 1>(key, lane);
    key = sort_step<32, 16>(key, lane);
    key = sort_step<32, 8>(key, lane);
    key = sort_step<32, 4>(key, lane);
    key = sort_step<32, 2>(key, lane);
    key = sort_step<32, 1>(key, lane);
    key = sort_step<64, 32>(key, lane);
    key = sort_step<64, 16>(key, lane);
    key = sort_step<64, 8>(key, lane);
    key = sort_step<64, 4>(key, lane);
    key = sort_step<64, 2>(key, lane);
    key = sort_step<64, 1>(key, lane);
    return key;
}

__device__ __forceinline__ void tree_paths_body(const UpdateArgs& a) {
    const uint32_t lane = threadIdx.x;
    // the entries: flags for the invalid ones, keys for the valid ones
    int64_t idx = -1;
    float p = -1.0f;
    if ((int64_t)lane < a.n) {
        idx = a.indices[lane];
        p = a.priorities[lane];
    }
    const bool have = (int64_t)lane < a.n;
    const bool idx_ok = idx >= 0 && idx < a.capacity, p_ok = valid_priority(p);
    if (__any(have && !idx_ok) && lane == 0) atomicOr(a.err, MRB_DERR_INDEX);
    if (__any(have && !p_ok) && lane == 0) atomicOr(a.err, MRB_DERR_PRIORITY);
    const bool valid = have && idx_ok && p_ok;
    const uint32_t key = bitonic_sort_wave(valid ? ((uint32_t)idx << 6) | lane : 0xffffffffu, lane);
    // this lane's entry from here on: the one the sort put here
    const bool mine = key != 0xffffffffu;
    const uint32_t leaf = key >> 6, pos = key & 63u;
    const uint32_t next_key = (uint32_t)__shfl_down((int)key, 1);
    bool act = mine && (lane == 63 || (next_key >> 6) != leaf || next_key == 0xffffffffu);  // the last entry aimed at the leaf
    uint32_t v = (uint32_t)a.leaves + leaf;  // heap index of the node this lane carries
    // siblings along the path, as memory holds them (level L's in [L - 1])
    float sib_s[kPathMaxDepth], sib_m[kPathMaxDepth];
#pragma unroll
    for (int L = kPathMaxDepth; L >= 1; --L) {
        sib_s[L - 1] = 0.0f;
        sib_m[L - 1] = 0.0f;
        if (L <= a.depth && act) {
            const uint32_t node = (v >> (a.depth - L)) ^ 1u;
            sib_s[L - 1] = a.sum[node];
            sib_m[L - 1] = a.mn[node];
        }
    }
    // the powers (every valid entry's counts for the running max, also one that loses its leaf)
    const float p_here = __shfl(p, (int)pos);
    const float q = mine ? powf_det(p_here, a.alpha) : 0.0f;
    const float qmax = wave_max(q);
    if (lane == 0 && qmax > 0.0f) raise_max(a.maxp, qmax);
    float cs = q, cm = q;
    if (act) {
        a.sum[v] = cs;
        a.mn[v] = cm;
    }
#pragma unroll
    for (int L = kPathMaxDepth; L >= 1; --L) {
        if (L <= a.depth) {  // wave-uniform
            const unsigned long long lanes = __ballot(act);
            const bool left = (v & 1u) == 0;
            const unsigned long long above = lanes & ~((2ull << lane) - 1ull), below = lanes & ((1ull << lane) - 1ull);
            const int nb = left ? (above ? __ffsll((long long)above) - 1 : -1) : (below ? 63 - __clzll((long long)below) : -1);
            const int src = nb < 0 ? (int)lane : nb;
            const uint32_t nv = (uint32_t)__shfl((int)v, src);
            const float ns = __shfl(cs, src), nm = __shfl(cm, src);
            const bool met = act && nb >= 0 && nv == (v ^ 1u);  // the other child is another entry's node
            const float os = met ? ns : sib_s[L - 1], om = met ? nm : sib_m[L - 1];
            cs = left ? cs + os : os + cs;
            cm = left ? fminf(cm, om) : fminf(om, cm);
            v >>= 1;
            if (met && !left) act = false;  // the left child's lane carries the parent
            if (act) {
                a.sum[v] = cs;
                a.mn[v] = cm;
            }
        }
    }
}

__global__ __launch_bounds__(64) void k_tree_paths(UpdateArgs a) { tree_paths_body(a); }

// ---------------------------------------------------------------------------
// A push of ONE row - the reference's insert() after every environment step - as one launch with one wave on
// the tree: the row's leaf and the `depth` nodes above it are all the call changes, and the other child of each
// is as memory holds it, at an address that follows from the slot. Lane L requests the sibling at level L, all
// at once; the walk from the leaf to the root is then a chain of additions and minima on values read from the
// lanes (no tile, no barrier, no second launch). The plain leading parameters are preloaded into scalar
// registers, so the requests go out when the wave starts. The row copy rides along as further workgroups.
// ---------------------------------------------------------------------------
constexpr int kPushOneMaxDepth = 30;

// The walk of one wave. kAfterUpdate: the walk follows an update_priorities in the same launch (same workgroup),
// so the running max is read where the update's atomic maxima were performed (past this compute unit's cache),
// and the siblings are requested only now, after the update's stores.
// `taken`: this launch moves the device's counters on, `ticket` holds them as the caller took them - the position is theirs,
// and, unless the caller has reported already (`report`), the wave's report (see counters_report) goes out behind the
// walk's own requests, so that nothing the walk waits for queues up behind the atomic.
template <bool kAfterUpdate>
__device__ __forceinline__ void push_one_walk(float* sum, float* mn, float* maxp, int64_t first_slot,
                                              int64_t capacity, int64_t leaves, int depth, float alpha,
                                              const float* priority, uint32_t* err, uint32_t lane,
                                              CounterTicket& ticket, bool taken, bool report, uint32_t readers) {
    // negative: the ring position is on the device (see Counters)
    const int64_t slot = taken             ? ticket_position(ticket, capacity)
                         : first_slot >= 0 ? first_slot
                                           : ring_position(counters_behind(err), capacity);
    const uint32_t v = (uint32_t)leaves + (uint32_t)slot;
    float sib_s = 0.0f, sib_m = 0.0f;
    if (lane >= 1 && lane <= (uint32_t)depth) {
        const uint32_t node = (v >> ((uint32_t)depth - lane)) ^ 1u;
        sib_s = sum[node];
        sib_m = mn[node];
    }
    // the leaf: the running max as the call finds it, or the given priority's power (an invalid one is flagged
    // and the row takes the running max, as a plain push would give it)
    const float running = kAfterUpdate ? __uint_as_float(__hip_atomic_load(reinterpret_cast<unsigned int*>(maxp), __ATOMIC_RELAXED,
                                                                           __HIP_MEMORY_SCOPE_AGENT))
                                       : *maxp;
    const float p = priority ? *priority : 0.0f;
    if (report) counters_report(ticket, err, readers, lane);
    const bool given = priority != nullptr && valid_priority(p);
    if (priority != nullptr && !given && lane == 0) atomicOr(err, MRB_DERR_PRIORITY);
    const float q = given ? powf_det_call(p, alpha) : running;
    float cs = q, cm = q;
    uint32_t node = v;
    if (lane == 0) {
        sum[node] = cs;
        mn[node] = cm;
    }
#pragma unroll
    for (int L = kPushOneMaxDepth; L >= 1; --L) {
        if (L <= depth) {  // wave-uniform
            const float os = lane_value(sib_s, L), om = lane_value(sib_m, L);
            const bool right = (node & 1u) != 0;
            cs = right ? os + cs : cs + os;
            cm = right ? fminf(om, cm) : fminf(cm, om);
            node >>= 1;
            if (lane == 0) {
                sum[node] = cs;
                mn[node] = cm;
            }
        }
    }
    // last: the leaf has read the running max as the call found it
    if (given && lane == 0 && q > 0.0f) raise_max(maxp, q);
}

// A workgroup of the row copy that rides along in such a launch. advance != 0: this launch moves the device's
// counters on, every wave reports its read of them (see counters_report).
__device__ __forceinline__ void push_rider(const PutArgs& put, uint32_t block, uint32_t* err, int64_t advance,
                                           int64_t capacity, uint32_t readers) {
    if (advance <= 0) {  // uniform over the launch
        rows_put_part(put, block, put.blocks);
        return;
    }
    const uint32_t lane = threadIdx.x & 63u;
    CounterTicket t = counters_take(err);
    counters_report(t, err, readers, lane);
    rows_put_part(put, block, put.blocks, ticket_position(t, capacity));
    counters_settle(t, err, advance, capacity, readers, lane);
}

// The tree wave of such a launch: the walk of push_one_walk, reporting its read of the device's counters (taken
// by the caller as `t` when advance != 0) beside the walk's own requests.
template <bool kAfterUpdate>
__device__ __forceinline__ void push_one_wave(float* sum, float* mn, float* maxp, int64_t first_slot, int64_t capacity,
                                              int64_t leaves, int depth, float alpha, const float* priority,
                                              uint32_t* err, uint32_t lane, CounterTicket& t, int64_t advance,
                                              uint32_t readers) {
    push_one_walk<kAfterUpdate>(sum, mn, maxp, first_slot, capacity, leaves, depth, alpha, priority, err, lane, t,
                                advance > 0, advance > 0, readers);
    if (advance > 0) counters_settle(t, err, advance, capacity, readers, lane);
}

template <bool kDev>
__global__ __launch_bounds__(kWG) void k_push_one(float* __restrict__ sum, float* __restrict__ mn, float* maxp,
                                                  int64_t first_slot, int64_t capacity, int64_t leaves, int depth,
                                                  float alpha, const float* priority, uint32_t* err, PutArgs put,
                                                  int64_t advance, uint32_t readers) {
    if (__builtin_expect(blockIdx.x >= 1, 0)) {  // (the tree workgroup's code comes first: it is the one the call waits for)
        if (kDev) push_rider(put, blockIdx.x - 1, err, advance, capacity, readers);
        else rows_put_part(put, blockIdx.x - 1, put.blocks);
        rider_ends();
    }
    if (threadIdx.x >= 64) return;
    CounterTicket t{};
    if (kDev) t = counters_take(err);
    push_one_wave<false>(sum, mn, maxp, first_slot, capacity, leaves, depth, alpha, priority, err, threadIdx.x, t,
                         kDev ? advance : 0, readers);
}

// ---------------------------------------------------------------------------
// update_priorities of at most 384 entries on a tree of at most 14 levels in ONE launch of ONE workgroup, a
// thread per entry, again along the entries' paths: a call then costs one launch instead of a leaf round and
// a top that wait for each other. What one wave settles among its lanes in k_tree_paths, the waves of a
// workgroup settle through LDS:
//   * the top kWgTopLevels + 1 levels of both trees (nodes [1, 4096), 32 KB) are staged in LDS when the
//     kernel starts; once the paths have reached them every lookup is a plain LDS read - LDS holds the
//     latest value of a node whether this call has changed it or not -, and the whole top is written back
//     at the end (recomputing a node this call has not touched reproduces its bits);
//   * below them the nodes this call changes are kept in LDS hash tables (node -> sum, min), one table per
//     step, three tables in rotation so that one can be cleared while another is read: a thread looks the
//     other nodes under its parent up there and takes memory's value - requested when the kernel starts,
//     the addresses follow from the leaf - for those the call has not changed;
//   * a step takes TWO levels: a thread combines its node with its sibling, the two children of the
//     parent's sibling with each other, and the two results into the grandparent - the same single rounded
//     sums and minima, in the same pairing, as a rebuild level by level - so a barrier is paid every other
//     level. Of the up to four changed nodes under a grandparent the lowest-numbered one's thread goes on
//     with it; the others stop (with consecutive slots in a call, hundreds of threads would otherwise hammer
//     one hash slot).
//   * entries aimed at one leaf elect the latest among them with a 64-bit LDS maximum of (position, p^alpha).
//   * a call of at most 64 entries (eight threads of the 512 per entry; at most 128 when launched with 1024) takes the levels below the staged top in ONE
//     step and without the rotating tables: lane j of an entry's cluster holds leaf j of the entry's group - memory's
//     value or, looked up in the election's table, the call's -, the cluster rebuilds the group's levels among its
//     lanes (exchanges inside a row of lanes) and puts the group's root into the staged top, where the entry's own
//     thread picks it up: two barrier steps of 0.7 us become one of 0.6.
// Why only small trees: every level below the staged top costs an entry six scattered 4-byte accesses to
// memory (sibling and cousins read, own node written, in both trees), and ONE compute unit moves about one
// such cache line per nanosecond. Measured per call: 10,000 leaves, 128 / 256 / 384 entries: 6.1 / 6.7 / 7.6 us
// against 8.1-8.3 us for the two launches; 2^17 leaves (six levels below the top): 8.2 / 9.7 / 11.6 us against
// 7.7; 2^20 leaves, 512 entries: 22 us against 8.7. On the small trees it also beats the one-wave kernel above
// for 64 entries or fewer (10,000 leaves: 5.45 against 5.87 us at 64, 5.15 against 5.82 at 16). The kernel itself
// handles up to 1024 entries and trees of kWgMaxDepth levels.
// ---------------------------------------------------------------------------
constexpr int kWgMaxEntries = 1024;
constexpr int kWgMinThreads = 512; // so that kWgPieces 16-byte pieces per thread stage the top of a tree
constexpr int kWgPieces = 2;
constexpr int kWgTopLevels = 11;                  // levels 0 .. 11 of both trees live in LDS
constexpr int kWgTopNodes = 2 << kWgTopLevels;    // 4096 (node 0 does not exist)
constexpr int kWgSlotsLog2 = 11;
constexpr int kWgSlots = 1 << kWgSlotsLog2;       // slots per hash table: twice the most entries
constexpr int kWgMaxDepth = 14;                  // deepest tree the kernel is compiled for
constexpr int kWgBestEntries = 384;              // most entries for which it beats two launches
constexpr int kWgHashSteps = (kWgMaxDepth - kWgTopLevels + 1) / 2;  // most two-level steps below the staged top
constexpr int kWgTopSteps = (kWgTopLevels + 1) / 2;

__device__ __forceinline__ uint32_t wg_hash(uint32_t node) { return (node * 2654435761u) >> (32 - kWgSlotsLog2); }

__device__ __forceinline__ unsigned long long wg_pack(float s, float m) {
    return ((unsigned long long)__float_as_uint(m) << 32) | __float_as_uint(s);
}

// The slot that holds `node`, claimed if no thread has claimed one yet (a table is never more than half full).
__device__ __forceinline__ uint32_t wg_claim(uint32_t* keys, uint32_t node) {
    uint32_t slot = wg_hash(node);
    for (;;) {
        const uint32_t old = atomicCAS(&keys[slot], 0u, node);
        if (old == 0u || old == node) return slot;
        slot = (slot + 1) & (kWgSlots - 1);
    }
}
// The same in two halves, for a caller with arithmetic to do while the first attempt is on its way: `found` is what
// wg_claim_first's attempt on the node's home slot returned.
__device__ __forceinline__ uint32_t wg_claim_first(uint32_t* keys, uint32_t node) {
    return atomicCAS(&keys[wg_hash(node)], 0u, node);
}
__device__ __forceinline__ uint32_t wg_claim_rest(uint32_t* keys, uint32_t node, uint32_t found) {
    uint32_t slot = wg_hash(node);
    while (!(found == 0u || found == node)) {
        slot = (slot + 1) & (kWgSlots - 1);
        found = atomicCAS(&keys[slot], 0u, node);
    }
    return slot;
}

// One probe of a lookup, its reads issued by the caller (so that several lookups' reads travel together):
// `key` and `val` are what the table holds at `slot`. Returns whether the call has changed `node`; then
// s and m receive its value, otherwise they keep what they hold (memory's value). kLeaf: the table is the
// election's, whose values are (position, p^alpha) and stand for sum and min alike.
template <bool kLeaf>
__device__ __forceinline__ bool wg_resolve(const uint32_t* keys, const unsigned long long* vals, uint32_t node,
                                           uint32_t slot, uint32_t key, unsigned long long val, float& s, float& m) {
    while (key != node) {
        if (key == 0u) return false;
        slot = (slot + 1) & (kWgSlots - 1);
        key = keys[slot];
        val = vals[slot];
    }
    s = __uint_as_float((uint32_t)val);
    m = kLeaf ? s : __uint_as_float((uint32_t)(val >> 32));
    return true;
}

// kTake: a push follows in the same kernel and moves the device's counters on: the workgroup's LAST wave - a call
// of a few dozen entries leaves it little else to do, while the first waves carry the entries - leaves them in
// `ticket` (requested behind the body's own first requests, see counters_take) and reports its read once the
// election is over, so that the report has long returned when the push looks at it (see counters_report).
// staged_s, staged_m: where the staged top of the two trees lies in LDS, for a caller that goes on using it (every
// node's latest value, nodes [1, 2 << min(depth, kWgTopLevels)), valid once the workgroup has passed a barrier).
// What a kernel that goes on after the update (k_tree_wg_push_sample) takes from it through LDS instead of
// reading memory again: the largest p^alpha of the update's entries, and the update's values of the nodes beside
// the path of the leaf that the kernel writes next - those below the staged top, where LDS does not hold the tree
// ([i]: the node i levels above the leaf level).
struct StepShared {
    uint32_t flags;  // MRB_DERR_* of the update's entries
    uint32_t qmax;   // as bits; 0: no valid entry
    uint32_t watch_set[4];
    float watch_s[4], watch_m[4];
    float leaf_value;  // (the other way: the written leaf's value, for the sample that follows)
    float max_w;       // the weights' common denominator, by a wave that does not sample
    // counters on the device: what the walking wave found there
    uint32_t watch_leaf;  // the leaf the caller writes next (else an argument of tree_wg_body)
    int64_t slot, size_after;
    uint64_t calls;
};

__device__ __forceinline__ void top_write_back(const UpdateArgs& a, const float* top_s, const float* top_m, uint32_t nthreads) {
    const int T = a.depth < kWgTopLevels ? a.depth : kWgTopLevels;
    const uint32_t top_vec = 1u << (T - 1);
#pragma unroll
    for (int j = 0; j < kWgPieces; ++j) {
        const uint32_t i = threadIdx.x + j * nthreads;
        if (i < top_vec) {
            reinterpret_cast<f32x4*>(a.sum)[i] = reinterpret_cast<const f32x4*>(top_s)[i];
            reinterpret_cast<f32x4*>(a.mn)[i] = reinterpret_cast<const f32x4*>(top_m)[i];
        }
    }
}
// The same by `count` threads of the workgroup, this one being number `index` among them.
__device__ __forceinline__ void top_write_back_by(const UpdateArgs& a, const float* top_s, const float* top_m, uint32_t index,
                                                  uint32_t count) {
    const int T = a.depth < kWgTopLevels ? a.depth : kWgTopLevels;
    const uint32_t top_vec = 1u << (T - 1);
#pragma unroll 4
    for (uint32_t i = index; i < top_vec; i += count) {
        reinterpret_cast<f32x4*>(a.sum)[i] = reinterpret_cast<const f32x4*>(top_s)[i];
        reinterpret_cast<f32x4*>(a.mn)[i] = reinterpret_cast<const f32x4*>(top_m)[i];
    }
}

// kStep: the caller goes on with the staged top and writes it back itself (top_write_back); `step` (zeroed by the
// caller before the workgroup's first barrier) receives what StepShared describes, watch_leaf being the heap
// number of the leaf the caller writes next - with kStep == 2 taken from `step` (left there before the first
// barrier: the caller had to read it from the device).
template <bool kTake, int kStep = 0, int kThreads = 0>
__device__ __forceinline__ void tree_wg_body(const UpdateArgs& a, CounterTicket& ticket, float*& staged_s, float*& staged_m,
                                             StepShared* step = nullptr, uint32_t watch_leaf = 0) {
    __shared__ __align__(16) float top_s[kWgTopNodes];
    __shared__ __align__(16) float top_m[kWgTopNodes];
    staged_s = top_s;
    staged_m = top_m;
    __shared__ __align__(16) uint32_t keys[3][kWgSlots];
    __shared__ __align__(16) unsigned long long vals[3][kWgSlots];
    // (kThreads: the caller's fixed number of threads - the launch's own is a read of the kernel-argument segment)
    const uint32_t tid = threadIdx.x, nthreads = kThreads ? (uint32_t)kThreads : blockDim.x, lane = tid & 63u;
    const int D = a.depth;                                // 2 .. kWgMaxDepth
    const int T = D < kWgTopLevels ? D : kWgTopLevels;    // the staged top ends at level T
    const int H = D - T;                                  // levels below it
    const int nh = (H + 1) >> 1, nt = (T + 1) >> 1;       // steps below and inside the top
    const int h_first = (H & 1) ? 1 : 2, t_first = (T & 1) ? 1 : 2;  // levels the first step of each kind takes
    // the entry
    const bool have = (int64_t)tid < a.n;
    int64_t idx = -1;
    float p = -1.0f;
    if (have) {
        idx = a.indices[tid];
        p = a.priorities[tid];
    }
    // A call of so few entries that eight threads can share one takes the levels below the staged top in ONE step
    // and without hash tables of its own: thread t is lane t & 7 of the cluster of entry t >> 3 and looks after
    // one leaf of the entry's group (the 2, 4 or 8 leaves under its ancestor at the staged top's lowest level).
    const bool clustered = H > 0 && (uint64_t)a.n * 8u <= nthreads;  // uniform
    const uint32_t ce = tid >> 3, cj = tid & 7u;
    int64_t cidx = -1;
    float cp = -1.0f;
    if (clustered && (int64_t)ce < a.n) {
        cidx = a.indices[ce];
        cp = a.priorities[ce];
    }
    // the running max as the kernel finds it, for the test that spares the atomic below (see raise_max; the max only
    // grows, so an older value spares no atomic that matters - and read now it is no round trip behind the power)
    // (a vector load: a scalar one would be waited for by the next barrier's wait for LDS)
    const float seen_max = __uint_as_float(__hip_atomic_load(reinterpret_cast<unsigned int*>(a.maxp), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
    // the top of both trees, on its way while the entries arrive
    const uint32_t top_vec = 1u << (T - 1);  // 16-byte pieces per tree: (2 << T) / 4, at most kWgPieces * kWgMinThreads
    f32x4 st_s[kWgPieces], st_m[kWgPieces];
#pragma unroll
    for (int j = 0; j < kWgPieces; ++j) {
        const uint32_t i = tid + j * nthreads;
        st_s[j] = 0.0f;
        st_m[j] = 0.0f;
        if (i < top_vec) {
            st_s[j] = reinterpret_cast<const f32x4*>(a.sum)[i];
            st_m[j] = reinterpret_cast<const f32x4*>(a.mn)[i];
        }
    }
    // empty tables (key 0 = free: no node has number 0) and election words
    {
        const f32x4 zero = 0.0f;
        for (uint32_t i = tid; i < 3 * kWgSlots / 4; i += nthreads) reinterpret_cast<f32x4*>(&keys[0][0])[i] = zero;
        for (uint32_t i = tid; i < kWgSlots / 2; i += nthreads) reinterpret_cast<f32x4*>(&vals[0][0])[i] = zero;
    }
    lds_barrier();
    const bool idx_ok = idx >= 0 && idx < a.capacity, p_ok = valid_priority(p);
    if (kStep) {  // (the caller raises the flags: it has not read the buffer's flag word's address yet)
        if (__any(have && !idx_ok) && lane == 0) atomicOr(&step->flags, (uint32_t)MRB_DERR_INDEX);
        if (__any(have && !p_ok) && lane == 0) atomicOr(&step->flags, (uint32_t)MRB_DERR_PRIORITY);
    } else {
        if (__any(have && !idx_ok) && lane == 0) atomicOr(a.err, MRB_DERR_INDEX);
        if (__any(have && !p_ok) && lane == 0) atomicOr(a.err, MRB_DERR_PRIORITY);
    }
    const bool valid = have && idx_ok && p_ok;
    const uint32_t leaf_node = (uint32_t)a.leaves + (uint32_t)(valid ? idx : 0);
    // memory's values of the nodes the steps below the top may need: requested now, used when the call has
    // not changed the node ([0] the sibling, [1] and [2] the children of the parent's sibling)
    float pre_s[kWgHashSteps][3], pre_m[kWgHashSteps][3];
#pragma unroll
    for (int s = 0; s < kWgHashSteps; ++s) {
#pragma unroll
        for (int c = 0; c < 3; ++c) {
            pre_s[s][c] = 0.0f;
            pre_m[s][c] = 0.0f;
        }
        if (s < nh && valid && !clustered) {
            const uint32_t v = leaf_node >> (s == 0 ? 0 : h_first + 2 * (s - 1));
            pre_s[s][0] = a.sum[v ^ 1u];
            pre_m[s][0] = a.mn[v ^ 1u];
            if (s > 0 || h_first == 2) {
                const uint32_t c0 = ((v >> 1) ^ 1u) << 1;
                pre_s[s][1] = a.sum[c0];
                pre_m[s][1] = a.mn[c0];
                pre_s[s][2] = a.sum[c0 | 1u];
                pre_m[s][2] = a.mn[c0 | 1u];
            }
        }
    }
    // (clustered: memory's value of this lane's leaf of its entry's group, both trees)
    const bool cvalid = clustered && cidx >= 0 && cidx < a.capacity && valid_priority(cp) && cj < (1u << H);
    const uint32_t cgroup = (((uint32_t)a.leaves + (uint32_t)(cvalid ? cidx : 0)) >> H) << H;  // the group's first leaf
    float cl_s = 0.0f, cl_m = 0.0f;
    if (cvalid) {
        cl_s = a.sum[cgroup + cj];
        cl_m = a.mn[cgroup + cj];
    }
    if (kTake && tid >= nthreads - 64) ticket = counters_take(a.err);
    // the election's first step: a slot for the entry's leaf (the attempt is on its way during the power)
    uint32_t found = 0;
    if (valid) found = wg_claim_first(keys[0], leaf_node);
    // the power, while all of that is on its way; every valid entry's counts for the running max, also that
    // of an entry that loses its leaf
    const float q = valid ? powf_det(p, a.alpha) : 0.0f;
    const float qmax = wave_max(q);
    if (lane == 0 && qmax > seen_max) atomicMax(reinterpret_cast<unsigned int*>(a.maxp), __float_as_uint(qmax));
    if (kStep && lane == 0 && qmax > 0.0f) atomicMax(&step->qmax, __float_as_uint(qmax));
    // the election: the latest entry aimed at a leaf owns it
    uint32_t slot = 0;
    if (valid) {
        slot = wg_claim_rest(keys[0], leaf_node, found);
        atomicMax(&vals[0][slot], ((unsigned long long)tid << 32) | __float_as_uint(q));
    }
    // the staged top goes into LDS (needed only after several more barriers)
#pragma unroll
    for (int j = 0; j < kWgPieces; ++j) {
        const uint32_t i = tid + j * nthreads;
        if (i < top_vec) {
            reinterpret_cast<f32x4*>(top_s)[i] = st_s[j];
            reinterpret_cast<f32x4*>(top_m)[i] = st_m[j];
        }
    }
    lds_barrier();
    if (kTake && tid >= nthreads - 64) counters_report(ticket, a.err, a.readers, lane);
    bool act = valid && (uint32_t)(vals[0][slot] >> 32) == tid;
    uint32_t v = leaf_node;
    float cs = q, cm = q;
    if (clustered) {
        // ---- below the staged top, a cluster per entry: every lane takes this call's value of its leaf where the
        // call changes it (the election's table holds every such leaf with the elected entry's power), the cluster
        // rebuilds the group's levels among its lanes and lane 0 goes on with the group's root. Clusters of entries
        // that share a group - or a leaf - do the same work and store the same bits.
        if (cvalid) {
            const uint32_t node = cgroup + cj, h = wg_hash(node);
            if (wg_resolve<true>(keys[0], vals[0], node, h, keys[0][h], vals[0][h], cl_s, cl_m)) {
                a.sum[node] = cl_s;
                a.mn[node] = cl_m;
            }
        }
        // (every lane takes part in the exchanges; lanes without a leaf hold values that go nowhere)
        const float s1 = cl_s + butterfly_peer<0>(cl_s), m1 = fminf(cl_m, butterfly_peer<0>(cl_m));
        const float s2 = s1 + butterfly_peer<1>(s1), m2 = fminf(m1, butterfly_peer<1>(m1));
        const float s3 = s2 + butterfly_peer<2>(s2), m3 = fminf(m2, butterfly_peer<2>(m2));
        if (cvalid) {
            if (H >= 2 && (cj & 1u) == 0) {
                a.sum[(cgroup + cj) >> 1] = s1;
                a.mn[(cgroup + cj) >> 1] = m1;
            }
            if (H == 3 && (cj & 3u) == 0) {
                a.sum[(cgroup + cj) >> 2] = s2;
                a.mn[(cgroup + cj) >> 2] = m2;
            }
            if (kStep) {
                if (kStep == 2) watch_leaf = step->watch_leaf;
                if ((watch_leaf >> H) << H == cgroup) {  // the group of the leaf the caller writes next: what lies beside its path
                    const uint32_t rel = watch_leaf - cgroup;
                    if (cj == (rel ^ 1u)) {
                        step->watch_s[0] = cl_s;
                        step->watch_m[0] = cl_m;
                        step->watch_set[0] = 1u;
                    }
                    if (H >= 2 && cj == (((rel >> 1) ^ 1u) << 1)) {
                        step->watch_s[1] = s1;
                        step->watch_m[1] = m1;
                        step->watch_set[1] = 1u;
                    }
                    if (H == 3 && cj == (((rel >> 2) ^ 1u) << 2)) {
                        step->watch_s[2] = s2;
                        step->watch_m[2] = m2;
                        step->watch_set[2] = 1u;
                    }
                }
            }
        }
        // The group's root goes into the staged top, and the ENTRY's thread takes the path from there (the entries'
        // threads sit in the first wave: the clusters' first lanes are spread over all of them, and a step inside the
        // top costs every wave that has a path to carry): it picks its node's value up behind the next barrier.
        if (cvalid && cj == 0) {
            top_s[cgroup >> H] = H == 3 ? s3 : H == 2 ? s2 : s1;
            top_m[cgroup >> H] = H == 3 ? m3 : H == 2 ? m2 : m1;
        }
        act = valid;  // (also an entry that lost its leaf to a later one: it carries the same values up the same path)
        v = leaf_node >> H;
    }
    // ---- below the staged top: the call's nodes in hash tables
#pragma unroll
    for (int s = 0; s < kWgHashSteps; ++s) {
        if (s < nh && !clustered) {  // uniform
            const uint32_t* kt = keys[s % 3];
            const unsigned long long* vt = vals[s % 3];
            const bool two = s > 0 || h_first == 2;
            const int up = s == 0 ? 0 : h_first + 2 * (s - 1);  // levels between v and the leaves
            if (kStep == 2) watch_leaf = step->watch_leaf;
            if (act) {
                a.sum[v] = cs;
                a.mn[v] = cm;
                if (kStep && (v ^ 1u) == (watch_leaf >> up)) {
                    step->watch_s[up] = cs;
                    step->watch_m[up] = cm;
                    step->watch_set[up] = 1u;
                }
                const uint32_t sib = v ^ 1u, c0 = ((v >> 1) ^ 1u) << 1, c1 = c0 | 1u;
                const uint32_t h0 = wg_hash(sib), h1 = wg_hash(c0), h2 = wg_hash(c1);
                const uint32_t k0 = kt[h0], k1 = two ? kt[h1] : 0u, k2 = two ? kt[h2] : 0u;
                const unsigned long long w0 = vt[h0], w1 = two ? vt[h1] : 0ull, w2 = two ? vt[h2] : 0ull;
                float os = pre_s[s][0], om = pre_m[s][0];
                const bool d_sib = s == 0 ? wg_resolve<true>(kt, vt, sib, h0, k0, w0, os, om)
                                          : wg_resolve<false>(kt, vt, sib, h0, k0, w0, os, om);
                const bool right = (v & 1u) != 0;
                float ps = right ? os + cs : cs + os, pm = right ? fminf(om, cm) : fminf(cm, om);
                if (!two) {
                    act = !(right && d_sib);
                    v >>= 1;
                    cs = ps;
                    cm = pm;
                } else {
                    float s0 = pre_s[s][1], m0 = pre_m[s][1], s1 = pre_s[s][2], m1 = pre_m[s][2];
                    const bool d0 = s == 0 ? wg_resolve<true>(kt, vt, c0, h1, k1, w1, s0, m0)
                                           : wg_resolve<false>(kt, vt, c0, h1, k1, w1, s0, m0);
                    const bool d1 = s == 0 ? wg_resolve<true>(kt, vt, c1, h2, k2, w2, s1, m1)
                                           : wg_resolve<false>(kt, vt, c1, h2, k2, w2, s1, m1);
                    const float us = s0 + s1, um = fminf(m0, m1);
                    const uint32_t par = v >> 1;
                    if (!(right && d_sib)) {  // the lower changed child stores the parent
                        a.sum[par] = ps;
                        a.mn[par] = pm;
                        if (kStep && (par ^ 1u) == (watch_leaf >> (up + 1))) {
                            step->watch_s[up + 1] = ps;
                            step->watch_m[up + 1] = pm;
                            step->watch_set[up + 1] = 1u;
                        }
                    }
                    const bool pright = (par & 1u) != 0;
                    cs = pright ? us + ps : ps + us;
                    cm = pright ? fminf(um, pm) : fminf(pm, um);
                    // the lowest-numbered changed node of the four goes on
                    act = !((right && d_sib) || (pright && (d0 || d1)));
                    v = par >> 1;
                }
            }
            // the table of the step before is free now: empty it for the step after the next
            if (s >= 1) {
                const f32x4 zero = 0.0f;
                for (uint32_t i = tid; i < kWgSlots / 4; i += nthreads) reinterpret_cast<f32x4*>(&keys[(s + 2) % 3][0])[i] = zero;
            }
            if (s + 1 < nh) {  // uniform
                if (act) {
                    const uint32_t at = wg_claim(keys[(s + 1) % 3], v);
                    vals[(s + 1) % 3][at] = wg_pack(cs, cm);
                }
                lds_barrier();
            }
        }
    }
    // ---- inside the staged top: LDS holds every node's latest value
#pragma unroll
    for (int u = 0; u < kWgTopSteps; ++u) {
        if (u < nt) {  // uniform
            if (act && !(clustered && u == 0)) {
                top_s[v] = cs;
                top_m[v] = cm;
            }
            lds_barrier();
            if (clustered && u == 0 && act) {
                cs = top_s[v];
                cm = top_m[v];
            }
            if (act) {
                const bool two = u > 0 || t_first == 2;
                const bool right = (v & 1u) != 0;
                const float os = top_s[v ^ 1u], om = top_m[v ^ 1u];
                const float ps = right ? os + cs : cs + os, pm = right ? fminf(om, cm) : fminf(cm, om);
                const uint32_t par = v >> 1;
                if (!two) {
                    cs = ps;
                    cm = pm;
                    v = par;
                } else {
                    const uint32_t c0 = (par ^ 1u) << 1;
                    const float us = top_s[c0] + top_s[c0 | 1u], um = fminf(top_m[c0], top_m[c0 | 1u]);
                    top_s[par] = ps;
                    top_m[par] = pm;
                    const bool pright = (par & 1u) != 0;
                    cs = pright ? us + ps : ps + us;
                    cm = pright ? fminf(um, pm) : fminf(pm, um);
                    v = par >> 1;
                }
            }
        }
    }
    if (act) {  // the root
        top_s[v] = cs;
        top_m[v] = cm;
    }
    // (kStep: the update's stores are performed before the caller's - to the same nodes, possibly - are issued)
    if (kStep) __builtin_amdgcn_s_waitcnt(0);
    lds_barrier();
    if (!kStep) top_write_back(a, top_s, top_m, nthreads);
}

// What the one-workgroup update needs first, as plain leading kernel parameters: those are preloaded into scalar
// registers, so the entries are requested when a wave starts, not a trip to the kernel-argument segment later
// (of three dependent trips - arguments, entries, the nodes beside the entries' leaves - the first goes away).
struct WgLead {
    const int64_t* indices;
    const float* priorities;
    float *sum, *mn, *maxp;
    int n, depth, capacity;
    float alpha;
};
#define MRB_WG_LEAD_PARAMS                                                                                      \
    const int64_t *__restrict__ lead_indices, const float *__restrict__ lead_priorities, float *lead_sum, float *lead_mn, \
        float *lead_maxp, int lead_n, int lead_depth, int lead_capacity, float lead_alpha
__device__ __forceinline__ UpdateArgs with_lead(const UpdateArgs& from, const WgLead& lead) {
    UpdateArgs a = from;
    a.indices = lead.indices;
    a.priorities = lead.priorities;
    a.sum = lead.sum;
    a.mn = lead.mn;
    a.maxp = lead.maxp;
    a.n = lead.n;
    a.depth = lead.depth;
    a.leaves = (int64_t)1 << lead.depth;
    a.capacity = lead.capacity;
    a.alpha = lead.alpha;
    return a;
}
#define MRB_WG_LEAD WgLead{lead_indices, lead_priorities, lead_sum, lead_mn, lead_maxp, lead_n, lead_depth, lead_capacity, lead_alpha}

__global__ __launch_bounds__(kWgMaxEntries) void k_tree_wg(MRB_WG_LEAD_PARAMS, UpdateArgs a_in) {
    const UpdateArgs a = with_lead(a_in, MRB_WG_LEAD);
    CounterTicket none{};
    float *top_s, *top_m;
    tree_wg_body<false>(a, none, top_s, top_m);
}

// ---------------------------------------------------------------------------
// update_priorities followed by a push of ONE row, in ONE launch (mrb_per_update_push: what a learner does after
// every step - the priorities of the batch it has just used, then the transition the actor has just produced).
// Workgroup 0 runs the one-workgroup (or one-wave) update above and then, behind a workgroup barrier, the walk
// of k_push_one: its waves share a compute unit, so the update's stores are what the walk's loads find. The
// row copy rides along as further workgroups, as in k_push_one.
//   slot      the pushed row's slot (negative: read from the device, see Counters)
//   priority  the pushed row's priority (NULL: the running max, which includes this call's update)
// ---------------------------------------------------------------------------
// kDev: the buffer's counters live on the device and this launch moves them on (see Counters); the other
// instantiation carries none of that.
template <bool kDev>
__global__ __launch_bounds__(kWgMaxEntries) void k_tree_wg_push(MRB_WG_LEAD_PARAMS, UpdateArgs a_in, int64_t slot,
                                                                const float* priority, PutArgs put) {
    if (__builtin_expect(blockIdx.x >= 1, 0)) {  // (the tree workgroup's code comes first: it is the one the call waits for)
        if (kDev) push_rider(put, blockIdx.x - 1, a_in.err, a_in.advance, a_in.capacity, a_in.readers);
        else rows_put_part(put, blockIdx.x - 1, put.blocks);
        rider_ends();
    }
    const UpdateArgs a = with_lead(a_in, MRB_WG_LEAD);
    // The device's counters are the last wave's business: it requests them among the update's first requests, hands
    // the position to the walking wave through LDS and moves the counters on while that wave walks.
    __shared__ int64_t s_position;
    const bool keeper = kDev && threadIdx.x >= blockDim.x - 64;
    CounterTicket t{};
    float *top_s, *top_m;
    tree_wg_body<kDev>(a, t, top_s, top_m);
    if (keeper && (threadIdx.x & 63u) == 0) s_position = ticket_position(t, a.capacity);
    __threadfence_block();
    __syncthreads();
    if (threadIdx.x < 64) {
        CounterTicket none{};
        if (kDev) {  // (the slot stays in scalar registers either way)
            const int64_t at = s_position;
            slot = ((int64_t)__builtin_amdgcn_readfirstlane((int)(at >> 32)) << 32) |
                   (uint32_t)__builtin_amdgcn_readfirstlane((int)at);
        }
        push_one_walk<true>(a.sum, a.mn, a.maxp, slot, a.capacity, a.leaves, a.depth, a.alpha, priority, a.err, threadIdx.x,
                            none, false, false, 0);
    } else if (keeper) {
        counters_settle(t, a.err, a.advance, a.capacity, a.readers, threadIdx.x & 63u);
    }
}
// ---------------------------------------------------------------------------
// A learner's whole step on a small buffer in ONE launch of ONE workgroup (mrb_per_update_push_sample): the
// priorities of the batch it has just used, the transition the actor has just produced, and the batch it uses
// next - update_priorities, insert and sample of the reference's loop (mindspore_rl/algorithm/dqn/dqn_trainer.py:76-87
// with the sample of the following iteration). Every one of the three is a launch of a few microseconds whose
// kernel works for a fraction of that; here the update's staged top of both trees stays in LDS, the walk of the
// pushed row reads and patches it there, and the sample's strata descend through it - a thread per stratum, three
// levels per LDS read, the levels below the staged top with one load from memory - and gather their rows.
// The workgroup copies the pushed row itself: the sample may pick it.
// The results are those of the three calls, bit for bit.
// ---------------------------------------------------------------------------
constexpr int kStepThreads = kWgMinThreads;  // threads of the kernel (1024 for an update of 65 to 128 entries: eight per entry); most strata
constexpr uint32_t kStepMaxPut = 2 * 64;  // most granules of the pushed row, which one wave copies
constexpr uint32_t kStepMaxGather = 64 * kStepThreads;  // most granules of the sampled batch

// A field table in LDS: the kernel-argument segment is not cached across launches, and a lookup in it by a thread's
// own field number is a memory round trip; two waves request the tables when the kernel starts and put them into
// LDS when the update is through.
struct LdsTable {
    uint8_t* store[MRB_MAX_FIELDS];
    uint8_t* io[MRB_MAX_FIELDS];
    uint32_t row_bytes[MRB_MAX_FIELDS], stride[MRB_MAX_FIELDS], units[MRB_MAX_FIELDS], vec_log2[MRB_MAX_FIELDS];
    uint64_t prefix[MRB_MAX_FIELDS + 1];
};

// Granule w of a table's work (fields one after the other, rows within a field, granules within a row): its field,
// row and byte offset in the row.
__device__ __forceinline__ int wg_locate(const LdsTable& l, int nfields, uint32_t w, uint32_t& row, uint32_t& off) {
    int f = 0;
    while (f + 1 < nfields && w >= (uint32_t)l.prefix[f + 1]) ++f;
    const uint32_t local = w - (uint32_t)l.prefix[f], units = l.units[f];
    row = local / units;
    off = (local - row * units) << l.vec_log2[f];
    return f;
}

// The walk of the pushed row's leaf to the root by one wave, lane L holding the sibling at level L as in
// push_one_walk - but nothing is read from memory after the update: the siblings inside the staged top are read
// in LDS, those below it were requested when the kernel started (sib_s, sib_m: memory's values BEFORE the update)
// and are replaced by the update's where it has changed them (StepShared); the running max is the one the kernel
// found (old_max) raised by the update's entries. Lane L ends up with the path's node at level L and stores it -
// inside the staged top to LDS only (the workgroup writes the top back), below it to memory -, the leaf's value is
// left in LDS for the sample. The sums are the chain of single additions from the leaf up (an addition gives the
// same bits whichever operand is the left child), one lane picking up each; the minima do not depend on the order
// they are taken in: lane L's is the least of the leaf and the siblings at the levels below L, a scan over the
// lanes of a row (depth <= kWgMaxDepth < 16).
// q: the leaf's value when the row comes with a valid priority of its own (`given`), else the running max is taken.
__device__ __forceinline__ void step_walk(const UpdateArgs& a, uint32_t leaf_node, uint32_t sib_node, float sib_s, float sib_m,
                                          float old_max, bool given, float q, float* top_s, float* top_m,
                                          uint32_t top_nodes, StepShared& step, uint32_t lane) {
    const int depth = a.depth;
    const bool holds = lane >= 1 && lane <= (uint32_t)depth;
    {
        // (every LDS read is issued whether its lane needs it or not, at an index made harmless: one round trip
        // instead of one per nested condition)
        const bool in_top = sib_node < top_nodes;
        const uint32_t at = in_top ? sib_node : 0u;
        const uint32_t up = holds && !in_top ? (uint32_t)depth - lane : 0u;  // at most kWgMaxDepth - kWgTopLevels - 1
        const float ts = top_s[at], tm = top_m[at];
        const uint32_t changed = step.watch_set[up];
        const float ws = step.watch_s[up], wm = step.watch_m[up];
        const uint32_t ub = step.qmax;
        if (holds) {
            sib_s = in_top ? ts : changed ? ws : sib_s;
            sib_m = in_top ? tm : changed ? wm : sib_m;
        }
        if (!given) {
            const uint32_t ob = __float_as_uint(old_max);
            q = __uint_as_float(ob > ub ? ob : ub);  // (non-negative floats order like their bits)
        }
    }
    if (lane == 0) step.leaf_value = q;
    // minima: y = the least sibling at this lane's level or below, then the lane above's y against the leaf
    const float inf = __builtin_inff();
    float y = holds ? sib_m : inf;
    y = fminf(y, row_lane_above<1>(y, inf));
    y = fminf(y, row_lane_above<2>(y, inf));
    y = fminf(y, row_lane_above<4>(y, inf));
    y = fminf(y, row_lane_above<8>(y, inf));
    const float cm = fminf(q, row_lane_above<1>(y, inf));
    // sums: lane L - 1 keeps the chain's value after the sibling at level L has been added
    float chain = q, cs = q;
#pragma unroll
    for (int L = kWgMaxDepth; L >= 1; --L) {
        if (L <= depth) {  // wave-uniform
            chain = chain + lane_value(sib_s, L);
            cs = lane == (uint32_t)(L - 1) ? chain : cs;
        }
    }
    if (lane <= (uint32_t)depth) {
        const uint32_t node = leaf_node >> ((uint32_t)depth - lane);
        if (node < top_nodes) {
            top_s[node] = cs;
            top_m[node] = cm;
        } else {
            a.sum[node] = cs;
            a.mn[node] = cm;
        }
    }
    if (given && lane == 0 && q > 0.0f) raise_max(a.maxp, q);
}

// What the kernel needs only when the update is through: read from the kernel-argument segment then, not before.
// (A scalar read of that segment ahead of a barrier would make the barrier's wait for LDS wait for the read as
// well - the two share a counter -, and the segment's first read is a memory round trip of a microsecond.)
struct StepLate {
    uint32_t* err;          // the buffer's flag word
    const float* priority;  // the pushed row's priority, or NULL: the running max
    const float* uniforms;  // the sample's draws, or NULL: the generator (seed, calls)
    int64_t* out_idx;
    float* out_w;
    int64_t size;           // rows stored once the row is pushed
    uint64_t seed, calls;
    float beta;
    IoTable put, get;       // the pushed row (io: the caller's row), the sampled batch (io: the caller's outputs)
};
// The kernel's arguments as the segment holds them.
struct StepKernarg {
    const int64_t* indices;
    const float* priorities;
    float *sum, *mn, *maxp;
    int slot_capacity, sizes;
    float alpha;
    StepLate late;
};
using StepKernargPtr = const __attribute__((address_space(1))) StepKernarg*;

// A read of the segment as a VECTOR load (`opaque_zero`: a zero the compiler cannot see through; with a uniform
// address it would make the load a scalar one): a scalar read in flight makes every wait for LDS - the next barrier,
// the next LDS read - wait for it too, the two share a counter.
template <typename T>
__device__ __forceinline__ T vector_read(const __attribute__((address_space(1))) T* p, uint32_t opaque_zero) {
    return *(p + opaque_zero);
}

__device__ __forceinline__ StepKernargPtr step_kernarg(bool not_before_here) {
    uint64_t bits = (uint64_t)__builtin_amdgcn_kernarg_segment_ptr();
    if (not_before_here) asm volatile("" : "+s"(bits));  // what is read through the result is requested after this point
    return (StepKernargPtr)bits;
}

// The sample, first half: a thread per stratum descends - through the staged top in LDS, three levels per read, and
// through the at most three levels below it with one load of the leaves under its node, among which the leaf
// written by this launch is replaced by its value from LDS (its store may still be on its way) - and leaves the
// slot in LDS. Returns the index; `picked` receives the leaf's value.
__device__ __forceinline__ int64_t wg_descend(const float* top_s, int top_levels, const float* sum, int depth, int64_t capacity,
                                              uint32_t batch, float u, uint32_t leaf_node, float leaf_value, float& picked,
                                              int64_t* s_slot) {
    const uint32_t tid = threadIdx.x;
    const float total = top_s[1];
    float mass = (u + (float)tid) * (total / (float)batch);  // each operation rounded once
    uint32_t node = 1;
    int d = 0;
    picked = total;
    while (d < top_levels) {  // uniform
        const int rest = top_levels - d, g = rest < 3 ? rest : 3;  // (four levels per read would be fewer reads and
                                                                   // more arithmetic: slower)
        if (g == 3) {
            const float4 lo = *reinterpret_cast<const float4*>(top_s + ((size_t)node << 3));
            const float4 hi = *reinterpret_cast<const float4*>(top_s + ((size_t)node << 3) + 4);
            node = (node << 3) + walk8(lo, hi, mass, picked);
        } else if (g == 2) {
            node = (node << 2) + walk4(*reinterpret_cast<const float4*>(top_s + ((size_t)node << 2)), mass, picked);
        } else {
            node = 2 * node + walk2(*reinterpret_cast<const float2*>(top_s + 2 * (size_t)node), mass, picked);
        }
        d += g;
    }
    const int g = depth - d;  // 0 .. kWgMaxDepth - kWgTopLevels
    if (g > 0) {
        const uint32_t first = node << g, at = leaf_node - first;  // (at: the written leaf's place among the loaded ones, if below 1 << g)
        if (g == 3) {
            float4 lo = *reinterpret_cast<const float4*>(sum + first), hi = *reinterpret_cast<const float4*>(sum + first + 4);
            lo.x = at == 0 ? leaf_value : lo.x;
            lo.y = at == 1 ? leaf_value : lo.y;
            lo.z = at == 2 ? leaf_value : lo.z;
            lo.w = at == 3 ? leaf_value : lo.w;
            hi.x = at == 4 ? leaf_value : hi.x;
            hi.y = at == 5 ? leaf_value : hi.y;
            hi.z = at == 6 ? leaf_value : hi.z;
            hi.w = at == 7 ? leaf_value : hi.w;
            node = first + walk8(lo, hi, mass, picked);
        } else if (g == 2) {
            float4 v = *reinterpret_cast<const float4*>(sum + first);
            v.x = at == 0 ? leaf_value : v.x;
            v.y = at == 1 ? leaf_value : v.y;
            v.z = at == 2 ? leaf_value : v.z;
            v.w = at == 3 ? leaf_value : v.w;
            node = first + walk4(v, mass, picked);
        } else {
            float2 v = *reinterpret_cast<const float2*>(sum + first);
            v.x = at == 0 ? leaf_value : v.x;
            v.y = at == 1 ? leaf_value : v.y;
            node = first + walk2(v, mass, picked);
        }
    }
    const int64_t idx = (int64_t)node - ((int64_t)1 << depth);
    s_slot[tid] = idx < capacity ? idx : capacity - 1;
    return idx;
}

// One granule of a copy: where it comes from, where it goes, its size.
struct GranulePlace {
    const gbyte* src;
    gbyte* dst;
    uint32_t vl;
};

// Sixteen 32-bit words are preloaded into scalar registers, two of them the segment's address: the fourteen leading
// parameters are what the update needs first (the numbers among them packed: slot_capacity = capacity << 16 | slot,
// sizes = n << 18 | batch << 8 | depth), so that its first requests go out when a wave starts.
// kDev: the buffer's counters live on the device (see Counters): the walking wave reads the ring position, the row
// count and the generator's call counter there when the kernel starts (they lie in front of the running max, whose
// address is preloaded), hands them to the others through LDS and stores them moved on; this one workgroup is the
// launch's only reader, so nobody has to be waited for. The other instantiation carries none of that.
// kThreads: 512, or 1024 for an update of 65 to 128 entries (eight threads per entry: tree_wg_body's one-step path).
template <bool kDev, int kThreads>
__global__ __launch_bounds__(kThreads) void k_tree_wg_push_sample(const int64_t* __restrict__ indices,
                                                                      const float* __restrict__ priorities, float* sum, float* mn,
                                                                      float* maxp, int slot_capacity, int sizes, float alpha,
                                                                      StepLate late_args) {
    __shared__ int64_t s_slot[kThreads];
    __shared__ LdsTable s_put, s_get;
    __shared__ StepShared s_step;
    const uint32_t tid = threadIdx.x, lane = tid & 63u;
    // the last wave holds none of the update's entries (n <= 384; lanes of a small call's clusters at most) and walks for
    // the push, the one before it copies the row and carries the two field tables
    const bool walker = tid >= kThreads - 64, putter = !walker && tid >= kThreads - 128;
    const int depth = sizes & 255;
    const uint32_t batch = ((uint32_t)sizes >> 8) & 1023u;
    int64_t slot = slot_capacity & 0xffff;  // (kDev: known to the walking wave first, to the others after the update)
    const int64_t capacity = (uint32_t)slot_capacity >> 16;
    const int top_levels = depth < kWgTopLevels ? depth : kWgTopLevels;
    const uint32_t top_nodes = 2u << top_levels;
    int64_t c_pushes = 0, c_size = 0, c_calls = 0;
    if (kDev && walker) {
        int64_t* const cnt = counters_before(maxp);
        c_pushes = __hip_atomic_load(cnt + kCntPushes, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        c_size = __hip_atomic_load(cnt + kCntSize, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        c_calls = __hip_atomic_load(cnt + kCntCalls, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        slot = __hip_atomic_load(cnt + kCntPos, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    uint32_t leaf_node = (1u << depth) + (uint32_t)slot;
    UpdateArgs a{};
    a.indices = indices;
    a.priorities = priorities;
    a.n = (uint32_t)sizes >> 18;
    a.sum = sum;
    a.mn = mn;
    a.maxp = maxp;
    a.depth = depth;
    a.leaves = (int64_t)1 << depth;
    a.capacity = capacity;
    a.alpha = alpha;
    // What depends on nothing before it is requested with the update's first loads: the tables (by vector loads, which
    // no barrier of the update waits for; held in registers until the update is through), the walking wave's view of
    // the tree below the staged top as the update finds it, and the few pointers the waves need as soon as the update
    // is through (vector loads as well: through an offset the compiler cannot see through, or it would make them
    // scalar ones).
    uint32_t opaque_zero = 0;
    asm volatile("" : "+v"(opaque_zero));
    const StepKernargPtr early = step_kernarg(false);
    const float* const uniforms = vector_read(&early->late.uniforms, opaque_zero);
    const float* priority = nullptr;
    uint32_t* err_early = nullptr;
    float sib_s = 0.0f, sib_m = 0.0f, old_max = 0.0f;
    uint32_t sib_node = 0;
    uint8_t *t_store = nullptr, *t_io = nullptr;
    uint32_t t_row_bytes = 0, t_stride = 0, t_units = 0, t_vec = 0;
    uint64_t t_prefix = 0;
    if (walker) {
        if (lane >= 1 && lane <= (uint32_t)depth) {
            sib_node = (leaf_node >> ((uint32_t)depth - lane)) ^ 1u;
            if (sib_node >= top_nodes) {
                sib_s = sum[sib_node];
                sib_m = mn[sib_node];
            }
        }
        old_max = __uint_as_float(__hip_atomic_load(reinterpret_cast<unsigned int*>(maxp), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
        priority = vector_read(&early->late.priority, opaque_zero);
        err_early = vector_read(&early->late.err, opaque_zero);
        if (lane < 4) s_step.watch_set[lane] = 0u;
        if (lane == 0) {
            s_step.qmax = 0u;
            s_step.flags = 0u;
            if (kDev) {
                s_step.watch_leaf = leaf_node;
                s_step.slot = slot;
                s_step.size_after = c_size + 1 < capacity ? c_size + 1 : capacity;
                s_step.calls = (uint64_t)c_calls;
            }
        }
    }
    const uint32_t t_lane = lane & 31u;  // (the wave before the last: lanes 0.. the pushed row's table, lanes 32.. the batch's)
    if (putter) {
        const __attribute__((address_space(1))) IoTable* t = lane >= 32 ? &early->late.get : &early->late.put;
        if (t_lane <= MRB_MAX_FIELDS) t_prefix = t->prefix[t_lane];
        if (t_lane < MRB_MAX_FIELDS) {
            t_store = t->store[t_lane];
            t_io = t->io[t_lane];
            t_row_bytes = t->row_bytes[t_lane];
            t_stride = t->stride[t_lane];
            t_units = t->units[t_lane];
            t_vec = t->vec_log2[t_lane];
        }
    }
    CounterTicket none{};
    float *top_s, *top_m;
    tree_wg_body<false, kDev ? 2 : 1, kThreads>(a, none, top_s, top_m, &s_step, leaf_node);  // (ends behind a barrier)
    if (kDev) {
        if (walker) {  // the counters moved on (this launch has no other reader of them)
            int64_t* const cnt = counters_before(maxp);
            if (lane == 0) {
                counters_store_advanced(cnt, c_pushes, c_size, slot, 1, capacity);
                if (!uniforms) cnt[kCntCalls] = c_calls + 1;
            }
        } else {
            slot = s_step.slot;
            leaf_node = (1u << depth) + (uint32_t)slot;
        }
    }
    if (putter) {
        LdsTable* mine = lane >= 32 ? &s_get : &s_put;
        if (t_lane <= MRB_MAX_FIELDS) mine->prefix[t_lane] = t_prefix;
        if (t_lane < MRB_MAX_FIELDS) {
            mine->store[t_lane] = t_store;
            mine->io[t_lane] = t_io;
            mine->row_bytes[t_lane] = t_row_bytes;
            mine->stride[t_lane] = t_stride;
            mine->units[t_lane] = t_units;
            mine->vec_log2[t_lane] = t_vec;
        }
    }
    // the strata's draws: needed a barrier from here
    float u = 0.0f;
    if (tid < batch && uniforms) u = ((const __attribute__((address_space(1))) float*)uniforms)[tid];
    if (walker) {  // from the pushed row's leaf to the root: first thing, the others wait for it
        float q = 0.0f;
        bool given = false;
        if (priority) {
            const float p = *(const __attribute__((address_space(1))) float*)priority;
            given = valid_priority(p);
            if (!given && lane == 0) atomicOr(err_early, MRB_DERR_PRIORITY);
            if (given) q = powf_det_call(p, alpha);
        }
        step_walk(a, leaf_node, sib_node, sib_s, sib_m, old_max, given, q, top_s, top_m, top_nodes, s_step, lane);
        if (lane == 0 && s_step.flags) atomicOr(err_early, s_step.flags);
    }
    // (behind the tables and the walk, i.e. behind every use of what was requested when the kernel started: a wave's
    // requests come back in order, and a wait for an old one that the compiler cannot tell from these would wait for these)
    asm volatile("" ::"v"(uniforms), "v"(u));
    const StepKernargPtr ka = step_kernarg(true);
    uint32_t* const err = vector_read(&ka->late.err, opaque_zero);
    const int put_fields = vector_read(&ka->late.put.nfields, opaque_zero), get_fields = vector_read(&ka->late.get.nfields, opaque_zero);
    const int64_t size = kDev ? s_step.size_after : vector_read(&ka->late.size, opaque_zero);
    const float beta = vector_read(&ka->late.beta, opaque_zero);
    const uint64_t seed = vector_read(&ka->late.seed, opaque_zero);
    const uint64_t calls = kDev ? s_step.calls : vector_read(&ka->late.calls, opaque_zero);
    int64_t* const out_idx = vector_read(&ka->late.out_idx, opaque_zero);
    float* const out_w = vector_read(&ka->late.out_w, opaque_zero);
    lds_barrier();
    // ---- the sample's descent; the other waves find their granules' places meanwhile
    const bool mine = tid < batch;
    const float total = top_s[1];
    float picked = total;
    int64_t idx = 0;
    if (mine) {
        if (!uniforms) u = rng_uniform(seed, calls, (uint64_t)tid);
        idx = wg_descend(top_s, top_levels, sum, depth, capacity, batch, u, leaf_node, s_step.leaf_value, picked, s_slot);
    }
    // the pushed row: the wave before the last requests its granules now and stores them at the end
    constexpr int kPutPer = kStepMaxPut / 64;
    AnyGranule put_granule[kPutPer];
    GranulePlace put_place[kPutPer];
    uint32_t put_work = 0;
    if (putter) {
        put_work = (uint32_t)s_put.prefix[put_fields];  // (its own writes to the table: no barrier needed)
#pragma unroll
        for (int j = 0; j < kPutPer; ++j) {
            const uint32_t w = lane + 64u * j;
            put_place[j].vl = 0;
            if (w < put_work) {
                uint32_t row, off;
                const int f = wg_locate(s_put, put_fields, w, row, off);  // (row is 0: one row)
                put_place[j].vl = s_put.vec_log2[f];
                put_place[j].dst = as_global(s_put.store[f]) + (uint64_t)slot * s_put.stride[f] + off;
                put_granule[j].load(as_global(s_put.io[f]) + off, put_place[j].vl);
            }
        }
    }
    // the weights' common denominator (pmin / total * size)^-beta: by the last wave, unless it holds strata itself
    const bool spare_wave = batch <= kThreads - 64;
    if (spare_wave && walker) {
        const float max_w = powf_det(top_m[1] / total * (float)size, -beta);
        if (lane == 0) s_step.max_w = max_w;
    }
    // the sampled rows by granule number over the batch, dealt to the threads behind the strata's waves first
    const uint32_t work = (uint32_t)s_get.prefix[get_fields];
    const uint32_t behind = (batch + 63u) & ~63u;
    const uint32_t w0 = tid >= behind ? tid - behind : tid + kThreads - behind;
    uint32_t row0 = 0, off0 = 0, vl0 = 0, stride0 = 0;
    int f0 = 0;
    gbyte* dst0 = nullptr;
    if (w0 < work) {
        f0 = wg_locate(s_get, get_fields, w0, row0, off0);
        vl0 = s_get.vec_log2[f0];
        stride0 = s_get.stride[f0];
        dst0 = as_global(s_get.io[f0]) + (uint64_t)row0 * s_get.row_bytes[f0] + off0;
    }
    lds_barrier();
    // Threads with neither a stratum nor a granule - whole waves of them on a small batch - write the tree's top back
    // while the others work (nothing below reads the top from memory); else everybody does at the end.
    const bool spare_back = behind + work + 64u <= (uint32_t)kThreads;
    if (spare_back && tid >= behind + work) top_write_back_by(a, top_s, top_m, tid - (behind + work), kThreads - (behind + work));
    // ---- the rows (a sampled row that is the pushed one is read where the push reads it: its store may still be on
    // its way), the weights while they are on their way, the outputs behind them
    AnyGranule first_granule;
    if (w0 < work) {
        const int64_t from = s_slot[row0];
        const gbyte* src = from == slot ? as_global(s_put.io[f0]) + off0 : as_global(s_get.store[f0]) + (uint64_t)from * stride0 + off0;
        first_granule.load(src, vl0);
    }
    float weight = 0.0f;
    if (mine) {
        const float max_w = spare_wave ? s_step.max_w : powf_det(top_m[1] / total * (float)size, -beta);
        weight = powf_det(picked / total * (float)size, -beta) / max_w;
    }
    if (w0 < work) first_granule.store(dst0, vl0);
    if (mine) {
        ((__attribute__((address_space(1))) int64_t*)out_idx)[tid] = idx;
        ((__attribute__((address_space(1))) float*)out_w)[tid] = weight;
        if (!(total > 0.0f) || total > 3.0e38f) atomicOr(err, MRB_DERR_TOTAL);
        if (idx >= size) atomicOr(err, MRB_DERR_UNFILLED);
    }
    for (uint32_t w = w0 + kThreads; w < work; w += kThreads) {
        uint32_t row, off;
        const int f = wg_locate(s_get, get_fields, w, row, off);
        const int64_t from = s_slot[row];
        const gbyte* src = from == slot ? as_global(s_put.io[f]) + off : as_global(s_get.store[f]) + (uint64_t)from * s_get.stride[f] + off;
        copy_granule(as_global(s_get.io[f]) + (uint64_t)row * s_get.row_bytes[f] + off, src, s_get.vec_log2[f]);
    }
    if (putter) {
#pragma unroll
        for (int j = 0; j < kPutPer; ++j)
            if (lane + 64u * j < put_work) put_granule[j].store(put_place[j].dst, put_place[j].vl);
    }
    if (!spare_back) top_write_back(a, top_s, top_m, kThreads);  // (last: its stores are ahead of no load)
}

template <bool kDev>
__global__ __launch_bounds__(kWG) void k_tree_paths_push(UpdateArgs a, int64_t slot, const float* priority, PutArgs put) {
    if (__builtin_expect(blockIdx.x >= 1, 0)) {  // (the tree workgroup's code comes first: it is the one the call waits for)
        if (kDev) push_rider(put, blockIdx.x - 1, a.err, a.advance, a.capacity, a.readers);
        else rows_put_part(put, blockIdx.x - 1, put.blocks);
        rider_ends();
    }
    if (threadIdx.x >= 64) return;
    CounterTicket t{};
    if (kDev) t = counters_take(a.err);
    tree_paths_body(a);
    __threadfence_block();
    push_one_wave<true>(a.sum, a.mn, a.maxp, slot, a.capacity, a.leaves, a.depth, a.alpha, priority, a.err, threadIdx.x, t,
                        kDev ? a.advance : 0, a.readers);
}

// ---------------------------------------------------------------------------
// Discounted return (mindspore_rl/utils/discounted_return.py:84-92): one thread per
// (batch, inner) column walks the time axis backwards; neighbouring threads hold
// neighbouring columns, so every step's loads and stores are coalesced. The loads do
// not depend on the recurrence, so they are issued UNROLL steps ahead of their use.
//   last = reward[t] + ((1 - done[t]) * gamma) * last, each operation rounded once.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kWG) void k_discounted_return(const float* __restrict__ reward,
                                                           const uint8_t* __restrict__ done,
                                                           const float* __restrict__ last_value,
                                                           float* __restrict__ out, int64_t timesteps, int64_t batch,
                                                           int64_t inner, float gamma) {
    constexpr int UNROLL = 32;
    const int64_t cols = batch * inner;
    const int64_t c = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (c >= cols) return;
    const int64_t b = c / inner;
    float last = last_value[c];
    int64_t t = timesteps - 1;
    for (; t >= UNROLL - 1; t -= UNROLL) {
        float r[UNROLL];
        uint32_t d[UNROLL];  // 32-bit: byte-sized register arrays make the compiler pack and unpack them
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            r[u] = __builtin_nontemporal_load(reward + (t - u) * cols + c);
            d[u] = done[(t - u) * batch + b];
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const float scaled = (1.0f - (d[u] ? 1.0f : 0.0f)) * gamma;
            last = r[u] + scaled * last;
            __builtin_nontemporal_store(last, out + (t - u) * cols + c);
        }
    }
    for (; t >= 0; --t) {
        const float scaled = (1.0f - (done[t * batch + b] ? 1.0f : 0.0f)) * gamma;
        last = reward[t * cols + c] + scaled * last;
        out[t * cols + c] = last;
    }
}

// The same recurrence for inputs with few columns, where a thread per column leaves the memory
// system idle: a workgroup takes 64 columns and walks the time axis backwards in chunks of
// kDrChunk steps through three LDS buffers, as a pipeline whose stages run at the same time on
// consecutive chunks:
//   deposit  waves 1..15 (the movers) put chunk s, requested a stage ago, into its LDS buffer ...
//   request  ... request chunk s+1's rewards and done flags into the registers just emptied
//            (independent, coalesced loads; they arrive during the next stage) ...
//   drain    ... and write chunk s-2's results from LDS to memory, while ...
//   recur    ... wave 0 runs the recurrence over chunk s-1 out of LDS (lane = column).
// One barrier per stage; no wave waits for a load it has just issued. The memory system so sees
// loads and stores all the time, instead of a load phase, a phase without traffic and a store
// phase per chunk. The arithmetic and its order are those of k_discounted_return.
// Every mover issues the SAME number of loads and stores in every stage, without a branch around any of them: a
// row past the end of a short chunk is replaced by the chunk's last row (loaded twice, stored twice with the same
// value), a chunk past the end of the time axis by one row that is already cached, a column past the last one
// by the workgroup's first column. Only so can the compiler count what is in flight: with a branch per element
// it waited for EVERYTHING before each deposit - also for the next chunk's loads, issued a moment before -
// and every stage paid a full trip to memory (0.6 us per stage, a quarter of the kernel's time).
// (lds_barrier: here the next chunk's requests and the last chunk's results stay in flight across it.)

constexpr int kDrCols = 64;
constexpr int kDrWG = 1024;
constexpr int kDrMovers = kDrWG - 64;          // threads of waves 1..15
constexpr int kDrSweep = kDrMovers / kDrCols;  // rows the movers cover at once
constexpr int kDrPer = 4;                      // elements a mover carries per chunk
constexpr int kDrChunk = kDrPer * kDrSweep;    // 60 steps; three buffers of 60 x 64 x 8 B are 92 KB of LDS
constexpr int kDrAhead = 3;                    // chunks on their way from memory at any time
__global__ __launch_bounds__(kDrWG) void k_discounted_return_tiled(const float* __restrict__ reward,
                                                                 const uint8_t* __restrict__ done,
                                                                 const float* __restrict__ last_value,
                                                                 float* __restrict__ out, int64_t timesteps,
                                                                 int64_t batch, int64_t inner, float gamma) {
    // per element: .x the reward in, the return out; .y the factor (1 - done) * gamma, put there by the mover that
    // holds the done flag, so that a step of the recurrence is one LDS read, one multiply-add, one LDS write
    __shared__ float2 s_val[3][kDrChunk * kDrCols];
    const int64_t cols = batch * inner;
    // Workgroups are dealt to the chip's eight dies in turn, and each die has its own L2. A workgroup's 64 done flags
    // of a time step are half a cache line, the neighbouring columns' workgroup reads the other half: with
    // neighbours on different dies every such line is fetched from memory twice (measured: 98.5 MB fetched per
    // launch for 81.9 MB of input at [1000, 16384]). So neighbouring column groups go to the SAME die: workgroup b
    // takes group (b mod 8) * (n / 8) + b / 8 when the grid divides by eight.
    uint32_t group = blockIdx.x;
    if ((gridDim.x & 7u) == 0) group = (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
    const int64_t c0 = (int64_t)group * kDrCols;
    const int ncols = (int)(cols - c0 < kDrCols ? cols - c0 : kDrCols);
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const bool mover = wave != 0;
    // a mover's elements of a chunk: column m % 64 of the rows m / 64, m / 64 + 15, ... (960 movers = 15 rows
    // of 64 columns per sweep)
    const int m = (int)threadIdx.x - 64;
    const int mrow = m / kDrCols;                                   // wave-uniform
    const int mcol = m % kDrCols < ncols ? m % kDrCols : 0;         // a column past the end doubles column 0
    const int64_t mb = (c0 + mcol) / inner;                         // the column's batch entry (done flags)
    const int nchunks = (int)((timesteps + kDrChunk - 1) / kDrChunk);
    // chunk c covers the steps [lo, lo + steps), counted from the end of the time axis; past the end: one row
    auto chunk_lo = [&](int c) -> int64_t {
        const int64_t hi = timesteps - (int64_t)c * kDrChunk;
        return hi > kDrChunk ? hi - kDrChunk : 0;
    };
    auto chunk_steps = [&](int c) -> int {
        const int64_t hi = timesteps - (int64_t)c * kDrChunk;
        return (int)(hi > kDrChunk ? kDrChunk : hi > 0 ? hi : 1);
    };
    // (1 - done) * gamma has two values, computed once
    const float scaled_live = (1.0f - 0.0f) * gamma, scaled_done = (1.0f - 1.0f) * gamma;
    // (done flags travel as 32-bit values: byte-sized register arrays make the compiler pack and unpack them)
    // kDrAhead register sets take turns: chunk c travels in set c % kDrAhead, requested kDrAhead stages before it
    // is deposited, so that several chunks are on their way at any time (one chunk in flight per compute unit is
    // less than the memory system needs to stay busy: it waited out a trip to memory per stage)
    float r[kDrAhead][kDrPer];
    uint32_t d[kDrAhead][kDrPer];
    auto request = [&](int c, float (&rr)[kDrPer], uint32_t (&dd)[kDrPer]) {
        const int64_t lo = chunk_lo(c);
        const int last_row = chunk_steps(c) - 1;
#pragma unroll
        for (int u = 0; u < kDrPer; ++u) {
            const int row = mrow + u * kDrSweep < last_row ? mrow + u * kDrSweep : last_row;  // wave-uniform
            rr[u] = __builtin_nontemporal_load(reward + (lo + row) * cols + c0 + mcol);
            dd[u] = done[(lo + row) * batch + mb];
        }
    };
    auto deposit = [&](int c, const float (&rr)[kDrPer], const uint32_t (&dd)[kDrPer]) {
        float2* dv = s_val[c % 3] + mrow * kDrCols + mcol;
#pragma unroll
        for (int u = 0; u < kDrPer; ++u) dv[u * kDrMovers] = make_float2(rr[u], dd[u] ? scaled_done : scaled_live);
    };
    auto drain = [&](int c) {
        const int64_t lo = chunk_lo(c);
        const int last_row = chunk_steps(c) - 1;
        const float2* src = s_val[c % 3] + mcol;
#pragma unroll
        for (int u = 0; u < kDrPer; ++u) {
            const int row = mrow + u * kDrSweep < last_row ? mrow + u * kDrSweep : last_row;  // wave-uniform
            __builtin_nontemporal_store(src[row * kDrCols].x, out + (lo + row) * cols + c0 + mcol);
        }
    };
    float last = 0.0f;
    if (wave == 0 && lane < ncols) last = last_value[c0 + lane];
    auto recur = [&](int c) {
        if (c >= nchunks || lane >= ncols) return;
        const int steps = chunk_steps(c);
        float2* val = s_val[c % 3];
        // 16 steps at a time through registers, so that the LDS reads are not serialised behind the
        // recurrence's stores
        constexpr int STEP = 15;
        int tt = steps - 1;
        for (; tt >= STEP - 1; tt -= STEP) {
            float2 v[STEP];
#pragma unroll
            for (int u = 0; u < STEP; ++u) v[u] = val[(tt - u) * kDrCols + lane];
#pragma unroll
            for (int u = 0; u < STEP; ++u) {
                last = v[u].x + v[u].y * last;
                v[u].x = last;
            }
#pragma unroll
            for (int u = 0; u < STEP; ++u) val[(tt - u) * kDrCols + lane].x = v[u].x;
        }
        for (; tt >= 0; --tt) {
            const float2 v = val[tt * kDrCols + lane];
            last = v.x + v.y * last;
            val[tt * kDrCols + lane].x = last;
        }
    };
    // stage s: the movers deposit chunk s, request chunk s + kDrAhead into the registers just emptied and drain
    // chunk s - 2; wave 0 runs the recurrence over chunk s - 1. The two roles run their own loops (the same number
    // of barriers each): the movers' loop then holds nothing but its own loads and stores, in fixed numbers.
    static_assert(kDrAhead >= 2, "the two stages without a drain use the first two register sets");
    if (!mover) {
        lds_barrier();
        for (int s = 1; s < nchunks + 2; ++s) {
            recur(s - 1);
            lds_barrier();
        }
        return;
    }
#pragma unroll
    for (int j = 0; j < kDrAhead; ++j) request(j, r[j], d[j]);
    deposit(0, r[0], d[0]);
    request(kDrAhead, r[0], d[0]);
    lds_barrier();
    deposit(1, r[1], d[1]);
    request(1 + kDrAhead, r[1], d[1]);
    lds_barrier();
    for (int s = 2; s < nchunks + 2; s += kDrAhead) {
#pragma unroll
        for (int j = 0; j < kDrAhead; ++j) {
            if (s + j >= nchunks + 2) break;  // (uniform; nothing is requested or stored after the loop)
            constexpr int kFirst = 2 % kDrAhead;
            const int set = (kFirst + j) % kDrAhead;  // = (s + j) % kDrAhead, known when the loop is unrolled
            deposit(s + j, r[set], d[set]);  // (past the end of the time axis: a row nobody reads, into a buffer nobody uses)
            request(s + j + kDrAhead, r[set], d[set]);
            drain(s + j - 2);
            lds_barrier();
        }
    }
}

// Device-resident counters (see Counters): after a push, and after a sample that used the generator.
__global__ void k_counters_advance(int64_t* counters, int64_t pushed, int64_t capacity, int64_t calls) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        if (pushed) counters_store_advanced(counters, counters[kCntPushes], counters[kCntSize], counters[kCntPos], pushed, capacity);
        counters[kCntCalls] += calls;
    }
}

// The uniform buffer's device-resident counters: [1] count, [2] the generator's call counter, [3] head, [4] the
// next write position. kUrb* name them; the row copy finds its position where a prioritized push finds it.
constexpr int kUrbWrite = kCntPos, kUrbCount = 1, kUrbCalls = 2, kUrbHead = 3;
constexpr int64_t kUrbDrawMax = 1 << 16;  // most rows a sample draws through the device-side index array

// count / head after an append of n rows (n <= capacity; the write position is chosen once per call: `count`
// while the buffer has never wrapped, else `head`), after a reset (n < 0), after `calls` generator-driven samples.
__global__ void k_urb_advance(int64_t* c, int64_t n, int64_t cap, int64_t calls) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    int64_t count = c[kUrbCount], head = c[kUrbHead];
    if (n < 0) {
        count = 0;
    } else if (n > 0) {
        if (count < cap && head == 0) {
            const int64_t room = cap - count;
            if (n <= room) {
                count += n;
            } else {
                count = cap;
                head = (n - room) % cap;
            }
        } else {
            head = (head + n) % cap;
            count = count + n < cap ? count + n : cap;
        }
    }
    c[kUrbCount] = count;
    c[kUrbHead] = head;
    c[kUrbWrite] = count < cap && head == 0 ? count : head;
    c[kUrbCalls] += calls;
}

// The slots of a generator-driven sample (uniform in [0, count), with replacement), or - logical >= -count -
// the slot of one logical position (0 = oldest, negative counts back from the newest), written out for a
// gather at given slots: with the counters on the device the gather cannot take them as arguments.
__global__ __launch_bounds__(kWG) void k_urb_slots(int64_t* dst, uint64_t seed, const int64_t* c, int64_t n,
                                                   int64_t logical, int one_item, uint32_t* err) {
    const int64_t i = (int64_t)blockIdx.x * kWG + threadIdx.x;
    if (i >= n) return;
    const int64_t count = c[kUrbCount], head = c[kUrbHead];
    if (!one_item) {
        dst[i] = count > 0 ? rng_below(seed, (uint64_t)c[kUrbCalls], (uint64_t)i, count) : 0;
        return;
    }
    int64_t at = logical < 0 ? logical + count : logical;
    if (at < 0 || at >= count) {
        atomicOr(err, MRB_DERR_INDEX);
        at = 0;
    }
    const int64_t t = count - head;
    dst[0] = at < t ? at + head : at - t;
}

// Fills a float array with one value (tree initialisation: sums 0, mins FLT_MAX).
// A kernel that does nothing: what one launch costs (mrb_bench_launch).
__global__ void k_nothing() {}

__global__ __launch_bounds__(kWG) void k_fill_f32(float* p, float v, uint64_t n) {
    const uint64_t stride = (uint64_t)gridDim.x * kWG;
    for (uint64_t i = (uint64_t)blockIdx.x * kWG + threadIdx.x; i < n; i += stride) p[i] = v;
}

}  // namespace mrb
