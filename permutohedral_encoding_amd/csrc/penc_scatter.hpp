// Scatter-add of (slot, value pair) contributions into one level's slice of the table gradient.
//
// What the memory system of gfx950 gives (measured with purpose-built probes):
//   * a global fp32 atomic costs one request per 64-byte segment touched by a wave instruction,
//     whatever the number of lanes in the segment (1..16), the scope or the footprint; the chip
//     retires about 21 G such requests/s.  A level with many distinct slots is therefore bound
//     by requests, not bytes.
//   * ds_add_f32 retires about one lane every 3 clocks per CU, whatever the addresses: 30 times
//     slower than integer LDS atomics (ds_add_u32, ds_cmpst_b32/b64) and plain LDS accesses, and
//     5-20 times slower than ds_add_f64 (1.5 lanes/clock when 8 addresses take all the traffic,
//     3 for random addresses, 7.5 without bank conflicts).
//
// Hence three stages, each taking what the previous one could not combine:
//   1. Accumulate cache in LDS.  Every workgroup keeps a small open-addressed table
//      (tag = slot) for the level it works on.  Coarse levels, where thousands of points share
//      a handful of vertices, are absorbed here completely; the table is flushed once at the end.
//      When the first tile shows that the level has only a few dozen distinct slots, the cache's
//      LDS is re-laid as one column of per-lane cells for each slot (column mode): lanes then
//      add without meeting each other, and the wave-wide folding that a handful of hot lines
//      needs, which is what bounds those levels (vector ALU), is not needed at all.
//   2. Slot-range bins (optional, needs a workspace).  A contribution that finds no line in the
//      cache is appended, as a record of 12 or 10 bytes, to the bin of its slot range (each workgroup has a
//      private segment in every bin, so appending costs one LDS counter increment and one
//      store); a second kernel (bin_reduce_kernel) reads each bin back coalesced, sums it in
//      LDS (fp64), and adds the range into the gradient with coalesced read-modify-writes.  This
//      turns the random scatter of the fine levels into streaming traffic.  A workgroup whose
//      look-up of the first tile's slots shows that the cache would not hit at its level never
//      fills it: the cache's LDS becomes staging space in which the records of a tile are sorted by
//      bin, so that records of one bin leave in runs of consecutive addresses (whole cache lines)
//      instead of one small store each.
//   3. Direct global atomics, with the two features of a slot in one instruction (lane pairs),
//      for whatever is left: no workspace, capacity too large for binning, or a full bin.
// The result never depends on a stage hitting: every stage falls through to the next.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "penc_lattice.hpp"

namespace penc {

constexpr uint32_t kDefaultDies = 8;   // accelerator dies (XCDs) of an MI355X, for when the runtime does not tell
constexpr int kBlock = 256;            // threads per workgroup of the gather-type kernels (4 wavefronts)
#ifndef PENC_SCATTER_BLOCK
#define PENC_SCATTER_BLOCK 512
#define PENC_SCATTER_TILES 8
#define PENC_SCATTER_TILES_LARGE 16
#define PENC_CACHE_LINES_LOG2 11
#endif
constexpr int kScatterBlock = PENC_SCATTER_BLOCK;  // threads per scattering workgroup (its wavefronts share one accumulate cache)
constexpr int kScatterTiles = PENC_SCATTER_TILES;  // tiles of kScatterBlock points a scattering workgroup walks (a "group" of points) ...
constexpr int kScatterTilesLarge = PENC_SCATTER_TILES_LARGE;  // ... or this many, when the launch still has workgroups to spare
constexpr int kCacheLinesLog2 = PENC_CACHE_LINES_LOG2;
constexpr int kCacheLines = 1 << kCacheLinesLog2;  // accumulate-cache lines per workgroup
constexpr int kWaveGroups = 6;         // same-slot groups a wave folds with DPP before it touches the cache
constexpr int kMinWaveGroup = 8;       // ... as long as the groups have at least this many lanes
constexpr int kColumnMinIdsLog2 = 5;   // column mode: the cache's kCacheLines cells per feature are 32 columns of 64 cells (one per lane) ...
#ifndef PENC_COLUMN_MAX_IDS_LOG2
#define PENC_COLUMN_MAX_IDS_LOG2 7
#endif
constexpr int kColumnMaxIdsLog2 = PENC_COLUMN_MAX_IDS_LOG2;   // ... up to 128 columns of 16 cells, by the number of distinct slots the first tile has shown
constexpr int kColumnProbes = 16;      // linear probes before a contribution gives up on the column table
enum ScatterMode : int { kModeCache = 0, kModeStream = 1, kModeColumns = 2 };
// vertices per thread a wave sorts by bin in one go (256 or 320 records): all D+1 of them up to D = 4
constexpr int stage_chunk(int pos_dim) { return pos_dim + 1 <= 4 ? 4 : 5; }
constexpr int kStageBins = 64;         // a wave counts one bin per lane: staging needs n_bins <= 64
constexpr int kWorkgroupSortMaxDim = 5;  // up to this input dimension a streaming workgroup sorts a tile's records across all its waves
constexpr int kBinSlotsLog2 = 13;      // slots per bin: 8192 (128 KiB of fp64 sums in LDS)
constexpr int kBinSlots = 1 << kBinSlotsLog2;
constexpr int kMaxBins = 512;          // bins per level
constexpr int kMaxBinSlotsLog2 = 16;   // tables of more than kMaxBins * kBinSlots slots (2^22) get bins of up to 2^16 slots, which their
                                       // reducer sums one range of kBinSlots slots after the other; above 2^25 slots nothing is binned
constexpr int kReduceBlock = 1024;     // threads of a bin_reduce_kernel workgroup

// A contribution on its way through a bin: the slot within the bin's range and the two values.
// In memory the records of a level are either one array of these 12-byte structures, or 10 bytes in
// two arrays indexed alike, the values (8 bytes) and the slots (2 bytes: a bin spans 2^13 slots).
// The fine levels move nothing but records through the HBM, twice, so the split form saves a sixth
// of their traffic (measured on a 2^18-slot table: the reducer 0.163 -> 0.150 ms, the scattering
// kernel unchanged); it takes two stores per record, which pays only where a tile's records leave in long
// runs, i.e. where the workgroup-wide sort of stream_tile applies (measured on a 2^22-slot table, whose runs are
// about four records: the scattering kernel 0.313 -> 0.355 ms, the reducer 0.207 -> 0.218 ms; at
// D = 8, whose waves sort on their own and leave runs of eight: 0.343 -> 0.356 ms, 0.137 -> 0.129 ms).
struct BinRecord {
    uint32_t slot_in_bin;
    float a0, a1;
};
static_assert(kBinSlotsLog2 <= 16, "a split record keeps its slot within the bin in 16 bits");
typedef float RecordValues __attribute__((ext_vector_type(2)));
typedef uint32_t RecordWords __attribute__((ext_vector_type(3), aligned(4)));
constexpr size_t kSplitRecordBytes = sizeof(RecordValues) + sizeof(uint16_t);

// Where the misses of the levels of one launch go.  Every scattering workgroup (a "group" of
// points at one level) owns a private segment of `segment_capacity` records in every
// bin, so appending needs no global atomics and no synchronisation: the cursor is an LDS counter.
//   records [level_in_pass][bin][group][segment_capacity]   12-byte records, or the 8-byte values of split ones
//   slots   [level_in_pass][bin][group][segment_capacity]   the 2-byte slots of split records; nullptr otherwise
//   counts  [level_in_pass][bin][group]            records actually written (<= segment_capacity)
//   direct  [level_in_pass][bin]                   nonzero once anything has been added into the gradient in the
//                                                  bin's slot range: straight from the scattering kernel (see
//                                                  GradSlice), or by the bin's reducer.  Cleared with the gradient, or,
//                                                  for a caller who keeps gradient and flags across calls (the sparse
//                                                  entry points), the caller's map of touched slot ranges.
// `records` == nullptr disables binning (`direct`, `n_bins` and `bin_shift` may still be set: flags without bins).
struct BinTarget {
    void* records;
    uint16_t* slots;
    uint32_t* counts;
    uint32_t* direct;
    uint32_t n_bins;
    uint32_t n_groups;
    uint32_t segment_capacity;
    uint32_t bin_shift;  // log2 of the slots per bin: kBinSlotsLog2, more only with more than kStageBins bins (whole records)
};

// `pass` describes the first level of a launch; level k of the launch follows k bin arrays later.
__device__ __forceinline__ BinTarget bins_of_level(const BinTarget& pass, uint32_t k) {
    BinTarget t = pass;
    if (pass.records != nullptr) {
        const size_t segments = static_cast<size_t>(k) * pass.n_bins * pass.n_groups;
        const size_t records = segments * pass.segment_capacity;
        t.records = static_cast<char*>(pass.records) + records * (pass.slots != nullptr ? sizeof(RecordValues) : sizeof(BinRecord));
        if (pass.slots != nullptr) t.slots += records;
        t.counts += segments;
    }
    if (pass.direct != nullptr) t.direct += static_cast<size_t>(k) * pass.n_bins;
    return t;
}

// Writes record `i` of a level (32-bit byte offsets: the host plans for that).
__device__ __forceinline__ void store_record(const BinTarget& bins, uint32_t i, uint32_t slot_in_bin, float a0, float a1) {
    char* const bytes = static_cast<char*>(bins.records);
    if (bins.slots != nullptr) {
        RecordValues v;
        v.x = a0;
        v.y = a1;
        *reinterpret_cast<RecordValues*>(bytes + i * static_cast<uint32_t>(sizeof(RecordValues))) = v;
        *reinterpret_cast<uint16_t*>(reinterpret_cast<char*>(bins.slots) + i * 2u) = static_cast<uint16_t>(slot_in_bin);
    } else {
        BinRecord rec;
        rec.slot_in_bin = slot_in_bin;
        rec.a0 = a0;
        rec.a1 = a1;
        *reinterpret_cast<BinRecord*>(bytes + i * static_cast<uint32_t>(sizeof(BinRecord))) = rec;
    }
}

// Record `i` of a bin whose first record is `first` (of the level's arrays), with ordinary loads.
template <bool kSplit>
__device__ __forceinline__ BinRecord load_record(const BinTarget& bins, size_t first, uint32_t i) {
    BinRecord rec;
    if constexpr (kSplit) {
        const RecordValues v = static_cast<const RecordValues*>(bins.records)[first + i];
        rec.slot_in_bin = bins.slots[first + i];
        rec.a0 = v.x;
        rec.a1 = v.y;
    } else {
        rec = static_cast<const BinRecord*>(bins.records)[first + i];
    }
    return rec;
}

// The same with the non-temporal hint: the reducer reads every record once, and a normal
// load would make room for it in the caches by evicting records the scatter has just written and
// that are still waiting there to be read (measured: the reducer of 2^18-slot tables 0.213 ->
// 0.168 ms; non-temporal *stores* of the records cost the scatter more than they save here).
template <bool kSplit>
__device__ __forceinline__ BinRecord load_record_once(const BinTarget& bins, size_t first, uint32_t i) {
    BinRecord rec;
    if constexpr (kSplit) {
        const RecordValues v = __builtin_nontemporal_load(static_cast<const RecordValues*>(bins.records) + first + i);
        rec.slot_in_bin = __builtin_nontemporal_load(bins.slots + first + i);
        rec.a0 = v.x;
        rec.a1 = v.y;
    } else {
        const RecordWords w = __builtin_nontemporal_load(reinterpret_cast<const RecordWords*>(static_cast<const BinRecord*>(bins.records) + first + i));
        const uint32_t w0 = w.x, w1 = w.y, w2 = w.z;  // copies first: a bit cast applied directly to a vector element reads element 0
        rec.slot_in_bin = w0;
        rec.a0 = __builtin_bit_cast(float, w1);
        rec.a1 = __builtin_bit_cast(float, w2);
    }
    return rec;
}

// One level's slice of the table gradient as the scatter sees it: a pair of features per slot,
// `slot_floats` floats from one slot to the next (2 when a level has two features; with four, the
// slice of features (0,1) or (2,3) of an array whose slots are four floats apart).
// `direct` (the level's BinTarget::direct, or nullptr without bins) is told about every add that goes
// straight into the gradient: a bin whose slot range received none still holds the zeros it was
// cleared to when its reducer workgroup arrives, which can then store its sums without reading
// the gradient first (on a 2^22-slot table, whose gradient no cache holds, that read is a third
// of the reducer's traffic).
struct GradSlice {
    float* base;
    uint32_t slot_floats;
    uint32_t* direct;
    uint32_t bin_shift;  // of the bins `direct` belongs to
    __device__ __forceinline__ float* at(uint32_t slot) const { return base + static_cast<size_t>(slot) * slot_floats; }
    // A plain store on purpose: many workgroups may set the same flag at once, all to 1, and nobody reads it before the
    // kernel has ended.  (As a relaxed atomic store of device scope, a store that writes through the L2, the levels that
    // sum in columns took up to 2.5 times as long and the kernel 8% longer.)
    __device__ __forceinline__ void mark_direct(uint32_t slot) const {
        if (direct != nullptr) direct[slot >> bin_shift] = 1u;
    }
};

__device__ __forceinline__ void global_add(float* addr, float v) {
    __hip_atomic_fetch_add(addr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum over the 64 lanes of a wavefront; the total is valid in lane 63.
__device__ __forceinline__ float wave_sum_to_last_lane(float v) {
    // row_shr:1,2,4,8 build the total of each row of 16 in its last lane (lanes shifted in from
    // outside the row read 0); row_bcast:15 adds it into rows 1 and 3, row_bcast:31 into rows 2 and 3
    constexpr int kShr1 = 0x111, kShr2 = 0x112, kShr4 = 0x114, kShr8 = 0x118, kBcast15 = 0x142, kBcast31 = 0x143;
#define PENC_DPP_ADD(CTRL, ROW_MASK) \
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true))
    PENC_DPP_ADD(kShr1, 0xf);
    PENC_DPP_ADD(kShr2, 0xf);
    PENC_DPP_ADD(kShr4, 0xf);
    PENC_DPP_ADD(kShr8, 0xf);
    PENC_DPP_ADD(kBcast15, 0xa);
    PENC_DPP_ADD(kBcast31, 0xc);
#undef PENC_DPP_ADD
    return v;
}

// The value `v` has in lane `lane` (wave-uniform index), broadcast to all lanes.
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Exclusive prefix sum over the 64 lanes of a wavefront; `total` is the sum of all lanes.
__device__ __forceinline__ uint32_t wave_exclusive_scan(uint32_t v, uint32_t& total) {
    // row_shr:1,2,4,8 scan each row of 16 (lanes shifted in from outside the row read 0);
    // row_bcast:15 adds the total of rows 0 and 2 to rows 1 and 3, row_bcast:31 that of rows 0-1 to rows 2-3
    int s = static_cast<int>(v);
    s += __builtin_amdgcn_update_dpp(0, s, 0x111, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x112, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x114, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x118, 0xf, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x142, 0xa, 0xf, true);
    s += __builtin_amdgcn_update_dpp(0, s, 0x143, 0xc, 0xf, true);
    total = static_cast<uint32_t>(__builtin_amdgcn_readlane(s, 63));
    return static_cast<uint32_t>(s) - v;
}

// Orders the LDS accesses of one wavefront: what its lanes wrote before is visible to all of them
// after (LDS executes a wave's instructions in order; this keeps the compiler from reordering them).
__device__ __forceinline__ void wave_lds_fence() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// Stage 3.  Lanes are paired (2p, 2p+1): first both lanes of a pair add the two features of the
// even lane's slot, then those of the odd lane's slot, so that each 8-byte slot is one request.
// Must be called with all 64 lanes of the wave active.
__device__ __forceinline__ void global_add_pairs(const GradSlice& level_grad, bool need, uint32_t slot,
                                                 float a0, float a1) {
    constexpr int kFromEven = 0xA0;  // quad_perm:[0,0,2,2]
    constexpr int kFromOdd = 0xF5;   // quad_perm:[1,1,3,3]
    if (need) level_grad.mark_direct(slot);
    const int odd = threadIdx.x & 1;
    const int slot_i = static_cast<int>(slot), need_i = need ? 1 : 0;
    const int a0_i = __builtin_bit_cast(int, a0), a1_i = __builtin_bit_cast(int, a1);
    {   // the even lane's contribution: even lane adds feature 0, odd lane feature 1
        const int s = __builtin_amdgcn_update_dpp(0, slot_i, kFromEven, 0xf, 0xf, true);
        const int n = __builtin_amdgcn_update_dpp(0, need_i, kFromEven, 0xf, 0xf, true);
        const int hi = __builtin_amdgcn_update_dpp(0, a1_i, kFromEven, 0xf, 0xf, true);
        const float v = __builtin_bit_cast(float, odd ? hi : a0_i);
        if (n) global_add(level_grad.at(static_cast<uint32_t>(s)) + odd, v);
    }
    {   // the odd lane's contribution
        const int s = __builtin_amdgcn_update_dpp(0, slot_i, kFromOdd, 0xf, 0xf, true);
        const int n = __builtin_amdgcn_update_dpp(0, need_i, kFromOdd, 0xf, 0xf, true);
        const int lo = __builtin_amdgcn_update_dpp(0, a0_i, kFromOdd, 0xf, 0xf, true);
        const float v = __builtin_bit_cast(float, odd ? a1_i : lo);
        if (n) global_add(level_grad.at(static_cast<uint32_t>(s)) + odd, v);
    }
}

// Folds runs of neighbouring lanes that add to the same slot, within each row of 16 lanes: a segmented
// inclusive scan over the row (DPP row shifts, four steps), after which the last lane of every run
// holds the run's sums and is the only one of it still `live`.  Batches whose consecutive points are
// neighbours in space (samples along a ray) make such runs at every level whose cells are wider than the
// sampling distance: left alone they are what LDS atomics are slowest at (a few lanes on each of many
// addresses, too few per address for the wave-wide fold below).  Returns the number of lanes folded away.
// Must be called with all 64 lanes of the wave active.  Worth its 45 instructions only where many lanes have such a
// neighbour: neighbours_share_slots() asks that of one vertex per tile, for all the tile's vertices.
__device__ __forceinline__ bool neighbours_share_slots(uint32_t slot, bool live) {
    const int key = live ? static_cast<int>(slot) : -1 - static_cast<int>(threadIdx.x & 63);
    const int prev = __builtin_amdgcn_update_dpp(0, key, 0x111 /* row_shr:1 */, 0xf, 0xf, true);
    return __popcll(__ballot((threadIdx.x & 15) != 0 && prev == key)) >= 16;
}
__device__ __forceinline__ uint32_t fold_adjacent_runs(uint32_t slot, bool& live, float& x0, float& x1) {
    constexpr int kShr1 = 0x111, kShl1 = 0x101;  // row_shr:1, row_shl:1; row_shr:n is 0x110 + n
    const uint32_t lane = threadIdx.x & 63, in_row = lane & 15;
    // a lane that adds nothing gets a key of its own, so it joins no run
    const int key = live ? static_cast<int>(slot) : -1 - static_cast<int>(lane);
    const int prev = __builtin_amdgcn_update_dpp(0, key, kShr1, 0xf, 0xf, true);
    // `open`: the partial sum of this lane does not reach back to the first lane of its run yet
    int open = (in_row != 0 && prev == key) ? 1 : 0;
#define PENC_SCAN_STEP(SHIFT)                                                                                              \
    {                                                                                                                      \
        const float s0 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x0), 0x110 + SHIFT, 0xf, 0xf, true)); \
        const float s1 = __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x1), 0x110 + SHIFT, 0xf, 0xf, true)); \
        const int so = __builtin_amdgcn_update_dpp(0, open, 0x110 + SHIFT, 0xf, 0xf, true);  /* 0 from beyond the row: a run ends there */      \
        x0 += open ? s0 : 0.0f;                                                                                            \
        x1 += open ? s1 : 0.0f;                                                                                            \
        open = open ? so : 0;                                                                                              \
    }
    PENC_SCAN_STEP(1)
    PENC_SCAN_STEP(2)
    PENC_SCAN_STEP(4)
    PENC_SCAN_STEP(8)
#undef PENC_SCAN_STEP
    const int next = __builtin_amdgcn_update_dpp(0, key, kShl1, 0xf, 0xf, true);
    const bool last_of_run = in_row == 15 || next != key;
    const bool was_live = live;
    live = live && last_of_run;
    return __popcll(__ballot(was_live && !live));
}

// LDS state of a scattering workgroup.  The accumulate cache sums in fp64 with ds_add_f64: its
// lines are hit by many lanes at once (that is what the cache is for), where a compare-and-swap
// loop degrades quadratically (measured: 10-40x slower on the coarsest levels) and ds_add_f32 is
// slow on this chip.  The fp64 partial sums are rounded to fp32 once, when the cache is flushed.
template <int kStageChunk>
struct ScatterStateT {
    static constexpr int kChunk = kStageChunk;
    static constexpr int kTail = (kScatterBlock / 64) * kStageChunk * 64 - kCacheLines;
    static_assert(kTail >= 0, "the staging slices cover the cache's values");
    int tag[kCacheLines];
    double val[2][kCacheLines];  // one array per feature: random lines then spread over all LDS bank pairs
    // when the workgroup streams, val and this tail together are its waves' staging slices
    uint4 stage_tail[kTail > 0 ? kTail : 1];
    uint32_t bin_count[kMaxBins];  // records this workgroup has appended to each bin so far
    uint32_t hits;                 // contributions the cache has absorbed into existing lines since the first tile
    // what the look-ups of the first tile's slots showed (see scatter_mode_decide)
    uint32_t wanted;               // contributions of the first tile
    uint32_t lines;                // lines they claimed: the tile's distinct slots, as far as the cache could take them
    uint32_t misses;               // contributions whose slot found no line
    uint32_t strangers;            // slots of the second tile that the first tile did not touch (counted for levels with few slots)
};

template <typename State>
__device__ __forceinline__ void scatter_begin(State& c) {
    for (int e = threadIdx.x; e < kCacheLines; e += kScatterBlock) {
        c.tag[e] = -1;
        c.val[0][e] = 0.0;
        c.val[1][e] = 0.0;
    }
    for (int b = threadIdx.x; b < kMaxBins; b += kScatterBlock) c.bin_count[b] = 0u;
    if (threadIdx.x == 0) {
        c.hits = 0u;
        c.wanted = 0u;
        c.lines = 0u;
        c.misses = 0u;
        c.strangers = 0u;
    }
    __syncthreads();
}

// Stage 2 for one contribution: append a record to this workgroup's segment of the slot's bin.
// Returns false when the segment is full.
template <typename State>
__device__ __forceinline__ bool append_record(State& c, const BinTarget& bins, uint32_t group, uint32_t slot,
                                              float a0, float a1) {
    const uint32_t b = slot >> bins.bin_shift;
    const uint32_t pos = atomicAdd(&c.bin_count[b], 1u);
    if (pos >= bins.segment_capacity) return false;
    store_record(bins, (b * bins.n_groups + group) * bins.segment_capacity + pos, slot & ((1u << bins.bin_shift) - 1u), a0, a1);
    return true;
}

// Looks `slot` up in the accumulate cache, claiming a free line if there is one.  Two candidate
// lines per slot (two-choice hashing): with one, a level with a few hundred distinct slots already
// loses several of them to collisions, and those are exactly the slots every wave keeps hitting.
// Returns the line, or -1 when both candidates belong to other slots; `found` tells whether the
// line already held the slot (a hit, as opposed to a claim).
// (Spreading the lanes that share a slot over replicated sub-tables, instead of folding them in
// registers first, was measured 30% slower on the coarse levels, and no faster on top of folding.)
template <int kProbes = 2, typename State>
__device__ __forceinline__ int cache_find(State& c, uint32_t slot, bool& found) {
    const int want = static_cast<int>(slot);
    int e = static_cast<int>(slot & (kCacheLines - 1));
    found = false;
    constexpr uint32_t kMix[3] = {0x9E3779B1u, 0x85EBCA6Bu, 0xC2B2AE35u};
    static_assert(kProbes >= 1 && kProbes <= 4, "one mixing constant per probe after the first");
#pragma unroll
    for (int probe = 0; probe < kProbes; ++probe) {
        int owner = c.tag[e];
        if (owner == want) {
            found = true;
            return e;
        }
        if (owner == -1) {
            owner = atomicCAS(&c.tag[e], -1, want);
            if (owner == -1 || owner == want) return e;
        }
        if (probe + 1 < kProbes) e = static_cast<int>((slot * kMix[probe]) >> (32 - kCacheLinesLog2));
    }
    return -1;
}

// Whether `slot` holds a line of the cache, without claiming one.
template <int kProbes = 2, typename State>
__device__ __forceinline__ bool cache_holds(const State& c, uint32_t slot) {
    const int want = static_cast<int>(slot);
    int e = static_cast<int>(slot & (kCacheLines - 1));
    constexpr uint32_t kMix[3] = {0x9E3779B1u, 0x85EBCA6Bu, 0xC2B2AE35u};
#pragma unroll
    for (int probe = 0; probe < kProbes; ++probe) {
        if (c.tag[e] == want) return true;
        if (probe + 1 < kProbes) e = static_cast<int>((slot * kMix[probe]) >> (32 - kCacheLinesLog2));
    }
    return false;
}

// Stage 2 for a whole tile once the workgroup streams (see scatter_mode_decide): the cache's LDS is
// staging space for a counting sort of the tile's records by bin, stage_chunk(D) vertices per thread
// at a time (2048 or 2560 records).  Every wave counts its records per bin (one LDS counter per
// bin and wave); the first wave turns the counts into run offsets (a bin's run is the waves' runs
// one after the other) and reserves room for each bin's run in the workgroup's segment with one
// add per bin; the waves lay their records out in that order in the staging space; and then all
// threads store the records in staging order: a wave instruction writes 64 consecutive records
// of (mostly) one bin, i.e. whole cache lines, where the records of a single wave would leave in
// runs of eight.  A staged record carries its destination (its index in the level's record
// array), so the store needs no search.  When a run does not fit its segment any more (rare: the
// segments hold the mean plus three standard deviations) the chunk checks every record against
// the room left and sends the excess to stage 3.
// Needs bins.n_bins <= kStageBins and a level's record array below 2^32 bytes (the host plans
// for both); all threads of the workgroup must call it together.
template <int D, typename State>
__device__ __forceinline__ void stream_tile(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                            uint32_t group, bool active, uvec<D + 1> slot, fvec<D + 1> a0,
                                            fvec<D + 1> a1) {
    constexpr int kWaves = kScatterBlock / 64;
    constexpr int kStageChunk = State::kChunk;
    static_assert(kCacheLines >= (3 * kWaves + 3) * 64, "the sort's index arrays live in the tag array");
    static_assert(offsetof(State, stage_tail) == offsetof(State, val) + sizeof(c.val) &&
                      (sizeof(c.val) + (State::kTail > 0 ? sizeof(c.stage_tail) : 0)) == kStageChunk * kScatterBlock * sizeof(uint4),
                  "val and stage_tail are one contiguous staging array");
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t* const words = reinterpret_cast<uint32_t*>(c.tag);
    uint32_t* const count = words + wave * 64;                  // [wave][bin] records of this wave per bin
    uint32_t* const offset = words + (kWaves + wave) * 64;      // [wave][bin] where the wave's run starts in the staging array
    uint32_t* const dest = words + (2 * kWaves + wave) * 64;    // [wave][bin] index of the run's first record in the level's record array
    uint32_t* const run_first = words + 3 * kWaves * 64;        // [bin] index of the workgroup's run for the bin
    uint32_t* const room = run_first + 64;                      // [bin] records the workgroup's segment can still take
    uint32_t* const header = room + 64;                         // [0] records staged, [1] whether every run fits
    uint4* const stage = reinterpret_cast<uint4*>(c.val);
    constexpr uint32_t kNoRoom = 0xFFFFFFFFu;
    constexpr int kChunks = (D + 1 + kStageChunk - 1) / kStageChunk;
    static_for<kChunks>(PENC_BODY(chunk) {
        PENC_INDEX(chunk);
        constexpr int kFirst = chunk * kStageChunk;
        constexpr int kCount = D + 1 - kFirst < kStageChunk ? D + 1 - kFirst : kStageChunk;
        count[lane] = 0u;
        wave_lds_fence();
        uvec<kStageChunk> place = 0u;  // rank of each record within its wave's run for the bin
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            if (active) place[j] = atomicAdd(&count[slot[kFirst + j] >> kBinSlotsLog2], 1u);
        });
        __syncthreads();
        if (wave == 0) {  // lane b looks after bin b
            uint32_t before[kWaves], mine = 0u;
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                before[w] = mine;
                mine += words[w * 64 + lane];
            }
            uint32_t total;
            const uint32_t first = wave_exclusive_scan(mine, total);
            const uint32_t taken = mine != 0u ? atomicAdd(&c.bin_count[lane], mine) : 0u;
            const uint32_t start = (lane * bins.n_groups + group) * bins.segment_capacity + taken;
            const bool all_fit = __all(taken + mine <= bins.segment_capacity);
#pragma unroll
            for (int w = 0; w < kWaves; ++w) {
                words[(kWaves + w) * 64 + lane] = first + before[w];
                words[(2 * kWaves + w) * 64 + lane] = start + before[w];
            }
            run_first[lane] = start;
            room[lane] = taken < bins.segment_capacity ? bins.segment_capacity - taken : 0u;
            if (lane == 0) {
                header[0] = total;
                header[1] = all_fit ? 1u : 0u;
            }
        }
        __syncthreads();
        const uint32_t total = header[0];
        const bool all_fit = header[1] != 0u;
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            if (active) {
                const uint32_t b = slot[kFirst + j] >> kBinSlotsLog2;
                // copies first: a bit cast applied directly to a vector element reads element 0
                const float v0 = a0[kFirst + j], v1 = a1[kFirst + j];
                const uint32_t to = dest[b] + place[j];
                uint4 e;
                e.x = slot[kFirst + j];
                e.y = __builtin_bit_cast(uint32_t, v0);
                e.z = __builtin_bit_cast(uint32_t, v1);
                e.w = all_fit || to - run_first[b] < room[b] ? to : kNoRoom;
                stage[offset[b] + place[j]] = e;
            }
        });
        __syncthreads();
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            const uint32_t i = j * kScatterBlock + threadIdx.x;
            bool spill = false;
            uint4 e = {0u, 0u, 0u, 0u};
            if (i < total) {
                e = stage[i];
                if (e.w != kNoRoom) {
                    store_record(bins, e.w, e.x & (kBinSlots - 1), __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
                } else {
                    spill = true;  // the segment is full: stage 3
                }
            }
            if (!all_fit && __any(spill))
                global_add_pairs(level_grad, spill, e.x, __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
        });
        // the next chunk (or tile) writes the counters after this wave's loads above and the staging
        // array after its next two barriers: nothing here is overwritten while another wave reads it
        wave_lds_fence();
    });
}

// The same sort for tables with more bins than a wave has lanes (up to one bin per thread of the
// workgroup: capacities up to 2^22).  One LDS counter per bin for the whole workgroup gives every
// record its place in the bin's run; thread b then looks after bin b: one block-wide prefix sum
// over the counts, one reservation per bin.  With hundreds of bins a tile leaves only a handful of
// records in each, but even runs of four records are worth it: appended one at a time, every
// 12-byte record is a store of its own to one of hundreds of open cache lines (measured on a
// 2^22-slot table: 42 us per level against 13 us for the sorted stores of a 2^18-slot one).
// The counters must be zero on entry (scatter_mode_decide clears them; every call leaves them so).
template <int D, typename State>
__device__ __forceinline__ void stream_tile_many(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                                 uint32_t group, bool active, uvec<D + 1> slot, fvec<D + 1> a0,
                                                 fvec<D + 1> a1) {
    constexpr int kWaves = kScatterBlock / 64;
    constexpr int kStageChunk = State::kChunk;
    static_assert(kMaxBins <= kScatterBlock, "one thread per bin");
    static_assert(kCacheLines >= 3 * kMaxBins + kWaves, "the sort's index arrays live in the tag array");
    const uint32_t wave = threadIdx.x >> 6;
    uint32_t* const words = reinterpret_cast<uint32_t*>(c.tag);
    uint32_t* const count = words;                       // [bin] records of this chunk
    uint32_t* const offset = words + kMaxBins;           // [bin] where the bin's run starts in the staging array
    uint32_t* const dest = words + 2 * kMaxBins;         // [bin] index of the run's first record in the level's record array
    uint32_t* const wave_total = words + 3 * kMaxBins;   // [wave] records of the wave's 64 bins
    uint4* const stage = reinterpret_cast<uint4*>(c.val);
    constexpr uint32_t kNoRoom = 0xFFFFFFFFu;
    constexpr int kChunks = (D + 1 + kStageChunk - 1) / kStageChunk;
    const uint32_t my_bin = threadIdx.x;  // the bin this thread looks after
    const uint32_t my_segment = (my_bin * bins.n_groups + group) * bins.segment_capacity;
    static_for<kChunks>(PENC_BODY(chunk) {
        PENC_INDEX(chunk);
        constexpr int kFirst = chunk * kStageChunk;
        constexpr int kCount = D + 1 - kFirst < kStageChunk ? D + 1 - kFirst : kStageChunk;
        uvec<kStageChunk> place = 0u;  // rank of each record within the workgroup's run for its bin
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            if (active) place[j] = atomicAdd(&count[slot[kFirst + j] >> bins.bin_shift], 1u);
        });
        __syncthreads();
        uint32_t mine = 0u;
        if (my_bin < bins.n_bins) {
            mine = count[my_bin];
            count[my_bin] = 0u;  // for the next chunk; nobody counts again before the barriers below
        }
        uint32_t in_wave;
        const uint32_t before_in_wave = wave_exclusive_scan(mine, in_wave);
        if ((threadIdx.x & 63) == 0) wave_total[wave] = in_wave;
        __syncthreads();
        uint32_t before = before_in_wave, total = 0u;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) {
            const uint32_t t = wave_total[w];
            before += w < static_cast<int>(wave) ? t : 0u;
            total += t;
        }
        bool fits = true;
        if (my_bin < bins.n_bins) {
            const uint32_t taken = c.bin_count[my_bin];  // only this thread touches its bin's cursor while the workgroup streams
            if (mine != 0u) c.bin_count[my_bin] = taken + mine;
            offset[my_bin] = before;
            dest[my_bin] = my_segment + taken;
            fits = taken + mine <= bins.segment_capacity;
        }
        const bool all_fit = __syncthreads_and(fits);
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            if (active) {
                const uint32_t b = slot[kFirst + j] >> bins.bin_shift;
                // copies first: a bit cast applied directly to a vector element reads element 0
                const float v0 = a0[kFirst + j], v1 = a1[kFirst + j];
                const uint32_t to = dest[b] + place[j];
                const uint32_t segment_end = (b * bins.n_groups + group + 1u) * bins.segment_capacity;
                uint4 e;
                e.x = slot[kFirst + j];
                e.y = __builtin_bit_cast(uint32_t, v0);
                e.z = __builtin_bit_cast(uint32_t, v1);
                e.w = all_fit || to < segment_end ? to : kNoRoom;
                stage[offset[b] + place[j]] = e;
            }
        });
        __syncthreads();
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            const uint32_t i = j * kScatterBlock + threadIdx.x;
            bool spill = false;
            uint4 e = {0u, 0u, 0u, 0u};
            if (i < total) {
                e = stage[i];
                if (e.w != kNoRoom) {
                    store_record(bins, e.w, e.x & ((1u << bins.bin_shift) - 1u), __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
                } else {
                    spill = true;  // the segment is full: stage 3
                }
            }
            if (!all_fit && __any(spill))
                global_add_pairs(level_grad, spill, e.x, __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
        });
        // the next chunk (or tile) counts into counters this chunk has cleared, overwrites offset/dest after its
        // first two barriers and the staging array after its third: nothing is overwritten while still read
    });
}

// The same sort with every wave on its own (no barriers), for the higher dimensions: their D+1
// vertices take two chunks, the waves of a workgroup drift apart over their longer tiles, and
// waiting for each other three times per chunk then costs more than the longer runs save
// (measured: 5-7% slower at D = 6, 7, 8; D = 5, whose second chunk is a single vertex, still gains 4%).
// The staging space is a 4 or 5 KiB slice per wave.  For stage_chunk(D) vertices per thread at a time, the wave
// counts its records per bin (one LDS counter per bin, owned by one lane), reserves room for each
// bin's run in the workgroup's segment with one add per bin, lays the records out bin by bin in
// its slice, and then stores them in that order: neighbouring lanes write neighbouring addresses.
// A staged record carries its destination (its index in the level's record array), so the
// store needs no search.  When a run does not fit its segment any more (rare: the segments hold
// the mean plus three standard deviations) the whole chunk takes the careful path, which checks
// every record against the room left and sends the excess to stage 3.
// Needs bins.n_bins <= kStageBins and a level's record array below 2^32 bytes (the host plans
// for both); all 64 lanes of the wave must call it together.
template <int D, typename State>
__device__ __forceinline__ void stream_tile_wave(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                            uint32_t group, bool active, uvec<D + 1> slot, fvec<D + 1> a0,
                                            fvec<D + 1> a1) {
    constexpr int kWaves = kScatterBlock / 64;
    constexpr int kStageChunk = State::kChunk;
    static_assert(kCacheLines / kWaves >= 4 * 64, "four 64-entry arrays per wave live in the tag array");
    static_assert(offsetof(State, stage_tail) == offsetof(State, val) + sizeof(c.val) &&
                      (sizeof(c.val) + (State::kTail > 0 ? sizeof(c.stage_tail) : 0)) / kWaves == kStageChunk * 64 * sizeof(uint4),
                  "val and stage_tail are one contiguous array of staging slices");
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    uint32_t* count = reinterpret_cast<uint32_t*>(c.tag) + wave * (kCacheLines / kWaves);  // records per bin
    uint32_t* offset = count + 64;  // where a bin's run starts in the wave's slice
    uint32_t* start = count + 128;  // index of the run's first record in the level's record array
    uint32_t* room = count + 192;   // records the workgroup's segment of the bin can still take
    uint4* stage = reinterpret_cast<uint4*>(c.val) + wave * (kStageChunk * 64);
    constexpr uint32_t kNoRoom = 0xFFFFFFFFu;
    constexpr int kChunks = (D + 1 + kStageChunk - 1) / kStageChunk;
    static_for<kChunks>(PENC_BODY(chunk) {
        PENC_INDEX(chunk);
        constexpr int kFirst = chunk * kStageChunk;
        constexpr int kCount = D + 1 - kFirst < kStageChunk ? D + 1 - kFirst : kStageChunk;
        count[lane] = 0u;
        wave_lds_fence();
        uvec<kStageChunk> place = 0u;  // rank of each record within its bin's run
        static_for<kCount>(PENC_BODY(j) {
            PENC_INDEX(j);
            if (active) place[j] = atomicAdd(&count[slot[kFirst + j] >> kBinSlotsLog2], 1u);
        });
        wave_lds_fence();
        // lane b looks after bin b: one reservation and one index computation per bin, not per record
        const uint32_t mine = count[lane];
        uint32_t total;
        offset[lane] = wave_exclusive_scan(mine, total);
        const uint32_t taken = mine != 0u ? atomicAdd(&c.bin_count[lane], mine) : 0u;
        start[lane] = (lane * bins.n_groups + group) * bins.segment_capacity + taken;
        const bool fits = taken + mine <= bins.segment_capacity;
        if (__all(fits)) {
            wave_lds_fence();
            static_for<kCount>(PENC_BODY(j) {
                PENC_INDEX(j);
                if (active) {
                    const uint32_t b = slot[kFirst + j] >> kBinSlotsLog2;
                    // copies first: a bit cast applied directly to a vector element reads element 0
                    const float v0 = a0[kFirst + j], v1 = a1[kFirst + j];
                    uint4 e;
                    e.x = slot[kFirst + j] & (kBinSlots - 1);
                    e.y = __builtin_bit_cast(uint32_t, v0);
                    e.z = __builtin_bit_cast(uint32_t, v1);
                    e.w = start[b] + place[j];
                    stage[offset[b] + place[j]] = e;
                }
            });
            wave_lds_fence();
            static_for<kCount>(PENC_BODY(j) {
                PENC_INDEX(j);
                const uint32_t i = j * 64 + lane;
                if (i < total) {
                    const uint4 e = stage[i];
                    store_record(bins, e.w, e.x, __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
                }
            });
        } else {
            room[lane] = taken < bins.segment_capacity ? bins.segment_capacity - taken : 0u;
            wave_lds_fence();
            static_for<kCount>(PENC_BODY(j) {
                PENC_INDEX(j);
                if (active) {
                    const uint32_t b = slot[kFirst + j] >> kBinSlotsLog2;
                    const float v0 = a0[kFirst + j], v1 = a1[kFirst + j];
                    uint4 e;
                    e.x = slot[kFirst + j];
                    e.y = __builtin_bit_cast(uint32_t, v0);
                    e.z = __builtin_bit_cast(uint32_t, v1);
                    e.w = place[j] < room[b] ? start[b] + place[j] : kNoRoom;
                    stage[offset[b] + place[j]] = e;
                }
            });
            wave_lds_fence();
            static_for<kCount>(PENC_BODY(j) {
                PENC_INDEX(j);
                const uint32_t i = j * 64 + lane;
                bool spill = false;
                uint4 e = {0u, 0u, 0u, 0u};
                if (i < total) {
                    e = stage[i];
                    if (e.w != kNoRoom) {
                        store_record(bins, e.w, e.x & (kBinSlots - 1), __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
                    } else {
                        spill = true;  // the segment is full: stage 3
                    }
                }
                if (__any(spill))
                    global_add_pairs(level_grad, spill, e.x, __builtin_bit_cast(float, e.y), __builtin_bit_cast(float, e.z));
            });
        }
        wave_lds_fence();
    });
}

// Column mode of stage 1, for a level whose points share a few dozen slots.  The cache's values
// are re-laid as 2^id_bits columns of kCacheLines >> id_bits cells; a slot owns a column (found
// through the first 2^id_bits tags, open addressing with linear probing) and a lane adds into the
// cell (lane mod cells) of its slot's column.  With 64 cells a lane meets no other lane of its
// wave, whatever the slots; with 32 or 16 cells two or four lanes share a cell.  The columns are
// summed when the level ends (column_flush).  Returns the column of `slot`, or -1 when the probes
// find only other slots (the contribution then takes stage 2 or 3 like any miss).
template <typename State>
__device__ __forceinline__ int column_find(State& c, uint32_t slot, uint32_t id_bits) {
    const int want = static_cast<int>(slot);
    const uint32_t mask = (1u << id_bits) - 1u;
    uint32_t e = (slot * 0x9E3779B1u) >> (32 - id_bits);
#pragma unroll 1
    for (int probe = 0; probe < kColumnProbes; ++probe) {
        int owner = c.tag[e];
        if (owner == want) return static_cast<int>(e);
        if (owner == -1) {
            owner = atomicCAS(&c.tag[e], -1, want);
            if (owner == -1 || owner == want) return static_cast<int>(e);
        }
        e = (e + 1u) & mask;
    }
    return -1;
}

template <int D, typename State>
__device__ __forceinline__ void column_tile(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                            uint32_t group, bool active, uint32_t id_bits, uvec<D + 1> slot,
                                            fvec<D + 1> a0, fvec<D + 1> a1) {
    const uint32_t cell_bits = kCacheLinesLog2 - id_bits;
    const uint32_t my_cell = threadIdx.x & ((1u << cell_bits) - 1u);
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        bool miss = active;
        if (active) {
            const int e = column_find(c, slot[r], id_bits);
            if (e >= 0) {
                const uint32_t cell = (static_cast<uint32_t>(e) << cell_bits) | my_cell;
                __hip_atomic_fetch_add(&c.val[0][cell], static_cast<double>(a0[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(&c.val[1][cell], static_cast<double>(a1[r]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                miss = false;
            }
        }
        if (miss && bins.records != nullptr) miss = !append_record(c, bins, group, slot[r], a0[r], a1[r]);
        if (__any(miss)) global_add_pairs(level_grad, miss, slot[r], a0[r], a1[r]);
    });
}

// Sums every column in use and adds the sums to the gradient (stage 3).  By all threads, between barriers.
template <typename State>
__device__ __forceinline__ void column_flush(State& c, const GradSlice& level_grad, uint32_t id_bits) {
    const uint32_t cell_bits = kCacheLinesLog2 - id_bits, cells = 1u << cell_bits;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    for (uint32_t id = wave; id < (1u << id_bits); id += kScatterBlock / 64) {
        const int owner = c.tag[id];  // the same for all lanes of the wave
        if (owner == -1) continue;
        double s0 = lane < cells ? c.val[0][(id << cell_bits) + lane] : 0.0;
        double s1 = lane < cells ? c.val[1][(id << cell_bits) + lane] : 0.0;
#pragma unroll
        for (int step = 32; step > 0; step >>= 1) {
            s0 += __shfl_xor(s0, step);
            s1 += __shfl_xor(s1, step);
        }
        if (lane == 0) {
            // straight into the gradient: a level in column mode leaves a few dozen sums per workgroup, and
            // as records they would only make every bin's reducer workgroup run for a handful of them
            float* g = level_grad.at(static_cast<uint32_t>(owner));
            level_grad.mark_direct(static_cast<uint32_t>(owner));
            global_add(g, static_cast<float>(s0));
            global_add(g + 1, static_cast<float>(s1));
        }
    }
}

// One tile's D+1 contributions per thread through stages 1-3.  All 64 lanes of every wave must
// call it together; `active` is false for lanes that carry no point (tail of the last tile), which
// only take part in the wave-wide steps.  `use_cache` (wave-uniform) is false once the workgroup
// has seen that the cache does not hit at this level; `mode` and `id_bits` are what
// scatter_mode_decide decided.  The return value is the number of hits of this wave in this tile.
template <int D, typename State>
__device__ __forceinline__ uint32_t scatter_tile(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                                 uint32_t group, bool active, bool use_cache, int mode, uint32_t id_bits,
                                                 uvec<D + 1> slot, fvec<D + 1> a0, fvec<D + 1> a1) {
    if (mode == kModeStream) {
        if (bins.n_bins > kStageBins) {
            stream_tile_many<D>(c, level_grad, bins, group, active, slot, a0, a1);
        } else if constexpr (D <= kWorkgroupSortMaxDim) {  // measured: the workgroup-wide sort wins up to D = 5, the per-wave one from D = 6 on
            stream_tile<D>(c, level_grad, bins, group, active, slot, a0, a1);
        } else {
            stream_tile_wave<D>(c, level_grad, bins, group, active, slot, a0, a1);
        }
        return 0u;
    }
    if (mode == kModeColumns) {
        column_tile<D>(c, level_grad, bins, group, active, id_bits, slot, a0, a1);
        return 0u;
    }
    uint32_t hits = 0;
    // (wave-uniform) the points of this tile follow each other in space: neighbouring lanes often add to the same slot
    const bool ordered = use_cache && neighbours_share_slots(slot[0], active);
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        float x0 = a0[r], x1 = a1[r];
        bool miss = active;
        if (use_cache) {
            // stage 1.  At the coarsest levels the 64 lanes of a wave hit two to six distinct slots,
            // and LDS atomics on one address serialise (about 5 clocks per lane): so first, up to
            // kWaveGroups times, take the slot of the first pending lane, sum the contributions of
            // all lanes that share it with DPP, and leave the sum with that lane alone.  A group
            // of fewer than kMinWaveGroup lanes means the wave's slots are spread out: stop.
            // neighbouring lanes on one slot first (points that follow each other in space), then the slots most of the wave shares
            if (ordered) hits += fold_adjacent_runs(slot[r], miss, x0, x1);
            unsigned long long pending = __ballot(miss);
#pragma unroll 1
            for (int round = 0; round < kWaveGroups && pending != 0ull; ++round) {
                const int leader = __builtin_ctzll(pending);
                const uint32_t leader_slot = __builtin_amdgcn_readlane(slot[r], leader);
                const bool in_group = miss && slot[r] == leader_slot;
                const unsigned long long members = __ballot(in_group);
                if (__popcll(members) < kMinWaveGroup) break;
                const float s0 = lane_value(wave_sum_to_last_lane(in_group ? x0 : 0.0f), 63);
                const float s1 = lane_value(wave_sum_to_last_lane(in_group ? x1 : 0.0f), 63);
                const bool is_leader = static_cast<int>(threadIdx.x & 63) == leader;
                x0 = is_leader ? s0 : x0;
                x1 = is_leader ? s1 : x1;
                miss = miss && (!in_group || is_leader);
                hits += __popcll(members) - 1;  // absorbed without touching the cache
                pending &= ~members;
            }
            bool found = false;
            if (miss) {
                // From D = 4 on a third candidate line: every contribution of a slot that finds no line becomes
                // a record, and tens of thousands of records on a handful of slots serialise in the LDS of
                // the one reducer workgroup that owns their bin.  At D = 3 the low 11 bits of a coarse level's
                // slots are all distinct and two candidates leave no slot out while the level fits; at D = 4
                // they collide (levels 6 and 7 of 24: 350 and 1000 slots, 4 and 110 of them left out; those
                // levels' reducer workgroups took 0.05-0.11 ms each, and with a third candidate the
                // double backward's table half went from 0.73 to 0.65 ms; at D = 3 it would add 2% to the
                // scattering kernel for nothing).
                constexpr int kProbes = D >= 4 ? 3 : 2;
                const int e = cache_find<kProbes>(c, slot[r], found);
                if (e >= 0) {
                    __hip_atomic_fetch_add(&c.val[0][e], static_cast<double>(x0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(&c.val[1][e], static_cast<double>(x1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    miss = false;
                }
            }
            hits += __popcll(__ballot(found));
        }
        // stage 2, then stage 3 for what stage 2 could not take
        if (miss && bins.records != nullptr) miss = !append_record(c, bins, group, slot[r], x0, x1);
        if (__any(miss)) global_add_pairs(level_grad, miss, slot[r], x0, x1);
    });
    return hits;
}

// The workgroup-wide decision whether stage 1 is worth its LDS traffic at this level: keep using the
// cache only while at least one contribution in `one_in` hits.  The evidence before tile `tile` is
// the look-up of the first tile's slots (a contribution that neither claimed a line nor missed
// would have hit) and the hits of the tiles processed since.  Against appending every miss to its
// bin on its own, one hit in eight pays; against sorting the tile's records by bin (stream_tile),
// which is cheaper than the cache's look-ups, it takes one in four.
template <int D, typename State>
__device__ __forceinline__ bool cache_pays(const State& c, int tile, uint32_t one_in = 8u) {
    const uint32_t settled = c.lines + c.misses;
    const uint32_t first_hits = c.wanted > settled ? c.wanted - settled : 0u;
    const uint32_t seen = c.wanted + static_cast<uint32_t>(tile > 1 ? tile - 1 : 0) * kScatterBlock * (D + 1);
    return (first_hits + c.hits) * one_in >= seen;
}

// Sends every line of the accumulate cache on to stage 2 (or 3).  By all threads, between barriers.
template <typename State>
__device__ __forceinline__ void cache_flush(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                            uint32_t group) {
    for (int e = threadIdx.x; e < kCacheLines; e += kScatterBlock) {
        const int owner = c.tag[e];
        if (owner != -1) {
            const float v0 = static_cast<float>(c.val[0][e]), v1 = static_cast<float>(c.val[1][e]);
            const bool binned = bins.records != nullptr && append_record(c, bins, group, static_cast<uint32_t>(owner), v0, v1);
            if (!binned) {
                float* g = level_grad.at(static_cast<uint32_t>(owner));
                level_grad.mark_direct(static_cast<uint32_t>(owner));
                global_add(g, v0);
                global_add(g + 1, v1);
            }
        }
    }
}

// Before the first tile is scattered (all threads call it, with the tile's slots): decides for the
// whole workgroup how the level goes.  The slots are looked up in the (empty) cache, which claims a
// line for every distinct slot as far as it can; the counts tell what the cache is good for.  One
// that would not hit is never filled: its LDS becomes staging space (kModeStream, see
// stream_tile; needs bins).  One that hits on at most 64 lines, and whose group of points is not expected to
// touch more than 96 slots in all, becomes columns (kModeColumns, `id_bits` says how many).  Otherwise the
// cache serves, with the lines already claimed.
template <int D, typename State, typename NextSlots>
__device__ __forceinline__ int scatter_mode_decide(State& c, const BinTarget& bins, bool active, uvec<D + 1> slot,
                                                   uint32_t& id_bits, bool next_active, NextSlots&& slots_of_next_tile,
                                                   int tiles_per_group) {
    uint32_t wanted = 0, missed = 0;  // over the wave
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        bool found = false;
        const bool miss = active && cache_find(c, slot[r], found) < 0;
        wanted += __popcll(__ballot(active));
        missed += __popcll(__ballot(miss));
    });
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&c.wanted, wanted);
        if (missed != 0u) atomicAdd(&c.misses, missed);
    }
    __syncthreads();  // every line the tile wants is claimed
    uint32_t used = 0;
    for (int e = threadIdx.x; e < kCacheLines; e += kScatterBlock) used += __popcll(__ballot(c.tag[e] != -1));
    if ((threadIdx.x & 63) == 0 && used != 0u) atomicAdd(&c.lines, used);
    // Columns are for a level whose few slots the whole group shares.  The first tile shows that when the points come in no
    // particular order; where they follow each other in space (every tile another ray, or the next stretch of a space-filling
    // curve) each tile brings slots of its own, the table of columns fills up, and every contribution that then finds no
    // column probes in vain and leaves one record.  The second tile's slots tell the two apart: how many of its contributions
    // go to slots the first tile did not touch?  (Asked only of a level that is a candidate for columns: the look at the
    // second tile costs a simplex search.)
    __syncthreads();
    const bool few_slots = cache_pays<D>(c, 0) && c.lines <= (1u << (kColumnMaxIdsLog2 - 1));  // the table of columns starts at most half full
    if (few_slots && tiles_per_group > 1) {
        const uvec<D + 1> next_slot = slots_of_next_tile();
        uint32_t strangers = 0;
        static_for<D + 1>(PENC_BODY(r) {
            PENC_INDEX(r);
            strangers += __popcll(__ballot(next_active && !cache_holds(c, next_slot[r])));
        });
        if ((threadIdx.x & 63) == 0 && strangers != 0u) atomicAdd(&c.strangers, strangers);
        __syncthreads();
    }
    int mode = kModeCache;
    const bool can_stream = bins.records != nullptr && bins.n_bins <= static_cast<uint32_t>(kMaxBins);
    // The slots the group will have touched in the end: the first tile's, and from every later tile as many new ones as the
    // second tile brought, counted twice (a slot at the rim of what a tile covers gets fewer contributions than one inside).
    const uint32_t expected_slots =
        c.lines + (2u * c.lines * c.strangers * static_cast<uint32_t>(tiles_per_group - 1)) / (c.wanted != 0u ? c.wanted : 1u);
    if (can_stream && !cache_pays<D>(c, 0, 4u)) {
        mode = kModeStream;
        if (bins.n_bins > kStageBins) {  // stream_tile_many wants its per-bin counters cleared
            for (int e = threadIdx.x; e < kMaxBins; e += kScatterBlock) c.tag[e] = 0;
            __syncthreads();
        }
    } else if (few_slots && expected_slots <= (3u << (kColumnMaxIdsLog2 - 2))) {  // the largest table may end up three quarters full
        mode = kModeColumns;
        id_bits = kColumnMinIdsLog2;
        while ((1u << (id_bits - 1)) < expected_slots && id_bits < static_cast<uint32_t>(kColumnMaxIdsLog2)) ++id_bits;
        for (int e = threadIdx.x; e < kCacheLines; e += kScatterBlock) c.tag[e] = -1;  // now the table of columns
        __syncthreads();
    }
    return mode;
}

// After the last tile: flushes the accumulate cache or the columns (through the bins when there are
// any; a streaming workgroup has neither left) and publishes how many records this workgroup left in each
// bin.  Call once, by all threads.
template <typename State>
__device__ __forceinline__ void scatter_end(State& c, const GradSlice& level_grad, const BinTarget& bins,
                                            uint32_t group, int mode, uint32_t id_bits) {
    __syncthreads();
    if (mode == kModeCache) cache_flush(c, level_grad, bins, group);
    if (mode == kModeColumns) column_flush(c, level_grad, id_bits);
    if (bins.records == nullptr) return;
    __syncthreads();
    for (uint32_t b = threadIdx.x; b < bins.n_bins; b += kScatterBlock) {
        const uint32_t n = c.bin_count[b];
        bins.counts[static_cast<size_t>(b) * bins.n_groups + group] = n < bins.segment_capacity ? n : bins.segment_capacity;
    }
}

// Second kernel of stage 2: a workgroup sums the records of one (bin, level) in LDS (fp64,
// ds_add_f64: a few hot slots must not serialise the whole bin, which rules out a compare-and-swap
// loop) and adds the bin's slot range into the gradient.  gridDim.z workgroups share a bin, each
// taking a contiguous range of the scattering workgroups' segments (a launch over few levels would
// otherwise leave most of the chip idle).  Each wavefront takes whole segments, so its loads are
// contiguous.  With one workgroup per bin nothing else touches the bin's slots while this kernel
// runs (the scattering kernel before it has completed, and bins do not overlap), so the final add is
// a plain coalesced read-modify-write; workgroups that share a bin add with atomics (consecutive
// addresses: one request per 64 bytes).
template <bool kSplit>  // whether the records are split (the host knows: BinTarget::slots)
__global__ void __launch_bounds__(kReduceBlock)
bin_reduce_kernel(BinTarget pass_bins, const float* __restrict__ window, uint32_t capacity, uint32_t feat_pairs,
                  float* __restrict__ table_grad, int first_level) {
    // one array per feature: lanes that hit different slots then spread over all bank pairs (interleaved
    // features would leave every other pair idle in each of the two adds)
    __shared__ double acc0[kBinSlots];
    __shared__ double acc1[kBinSlots];
    const uint32_t bin = blockIdx.x;
    // last level first: with the usual coarse-to-fine level list the bins with the most records are
    // started first and the nearly empty ones fill the tail of the launch
    const uint32_t level_in_pass = gridDim.y - 1 - blockIdx.y;
    // with more than two features per level, every pair of features is scattered and reduced like a level of its own
    const uint32_t pair_level = static_cast<uint32_t>(first_level) + level_in_pass;
    const uint32_t level = pair_level / feat_pairs, pair = pair_level % feat_pairs;
    if (window[level] == 0.0f) return;  // masked level: its scattering workgroups wrote no counts
    const BinTarget bins = bins_of_level(pass_bins, level_in_pass);
    constexpr uint32_t kWaves = kReduceBlock / 64;
    constexpr uint32_t kUnroll = 4;  // even
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const uint32_t per_split = (bins.n_groups + gridDim.z - 1) / gridDim.z;
    const uint32_t group_begin = blockIdx.z * per_split;
    const uint32_t group_end = group_begin + per_split < bins.n_groups ? group_begin + per_split : bins.n_groups;
    const uint32_t* counts = bins.counts + static_cast<size_t>(bin) * bins.n_groups;
    const size_t first = static_cast<size_t>(bin) * bins.n_groups * bins.segment_capacity;  // the bin's first record
    // A bin nothing was appended to (the levels whose scattering workgroups summed in columns, a slot
    // range no point touches) ends here: the look at the counts overlaps the clearing of the sums,
    // and the barrier that follows the clearing carries the vote.
    bool any = false;
    for (uint32_t g = group_begin + threadIdx.x; g < group_end; g += kReduceBlock) any = any || counts[g] != 0u;
    for (int s = threadIdx.x; s < kBinSlots; s += kReduceBlock) {
        acc0[s] = 0.0;
        acc1[s] = 0.0;
    }
    if (!__syncthreads_or(any)) return;
    // segments g = group_begin + wave, + kWaves, ...; their record counts are fetched 64 at a time
    // (one per lane) so that no segment has to wait for its own count.  The records are walked in
    // chunks of kUnroll wave-widths, and the next chunk's loads are issued before the current
    // chunk's LDS atomics, so a wave always has loads in flight.
    constexpr uint32_t kChunk = 64 * kUnroll;
    // Short segments (a large table has hundreds of bins, so a scattering workgroup leaves only a few
    // dozen records in each): a quarter of the wave per segment, four segments at a time, each taken
    // whole in one step of kShortUnroll loads per lane.
    constexpr uint32_t kShortLanes = 16, kShortUnroll = 8, kShortMax = kShortLanes * kShortUnroll;
    for (uint32_t g0 = group_begin + wave; g0 < group_end; g0 += kWaves * 64) {
        const uint32_t mine = g0 + lane * kWaves;
        const uint32_t my_count = mine < group_end ? counts[mine] : 0u;
        const uint32_t n_segments = (group_end - g0 + kWaves - 1) / kWaves < 64u ? (group_end - g0 + kWaves - 1) / kWaves : 64u;
        if (__ballot(my_count > kShortMax) == 0ull) {
            const uint32_t quarter = lane / kShortLanes, l = lane % kShortLanes;
            const uint32_t n_steps = (n_segments + 3) / 4;
            const auto fetch4 = [&](uint32_t step, BinRecord (&rec)[kShortUnroll]) {
                const uint32_t k = 4 * step + quarter;  // < 64; lanes past the last segment hold a count of 0
                const uint32_t count = static_cast<uint32_t>(__shfl(static_cast<int>(my_count), static_cast<int>(k)));
                const uint32_t seg = (g0 + k * kWaves) * bins.segment_capacity;  // within the bin: below 2^29 like the level's records
#pragma unroll
                for (uint32_t u = 0; u < kShortUnroll; ++u) {
                    const uint32_t i = u * kShortLanes + l;
                    // (normal loads: neighbouring short segments share cache lines)
                    rec[u] = load_record<kSplit>(bins, first, i < count ? seg + i : 0u);  // the bin's first record stands in where there is none
                }
                return count;
            };
            BinRecord cur[kShortUnroll], next[kShortUnroll];
            uint32_t cur_count = fetch4(0, cur), next_count = 0;
            for (uint32_t step = 0; step < n_steps; ++step) {
                if (step + 1 < n_steps) next_count = fetch4(step + 1, next);
#pragma unroll
                for (uint32_t u = 0; u < kShortUnroll; ++u)
                    if (u * kShortLanes + l < cur_count) {
                        const uint32_t cell = cur[u].slot_in_bin;
                        __hip_atomic_fetch_add(&acc0[cell], static_cast<double>(cur[u].a0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        __hip_atomic_fetch_add(&acc1[cell], static_cast<double>(cur[u].a1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
#pragma unroll
                for (uint32_t u = 0; u < kShortUnroll; ++u) cur[u] = next[u];
                cur_count = next_count;
            }
            continue;
        }
        const auto count_of = [&](uint32_t k) { return static_cast<uint32_t>(__builtin_amdgcn_readlane(my_count, k)); };
        // What a lane holds of one chunk, as loaded: split records are read two to a lane (16 bytes of
        // values, 4 of slots: a quarter of the load instructions) and taken apart only when they are
        // added, so that nothing between the loads and the previous chunk's adds waits for them.
        typedef float ValuePair __attribute__((ext_vector_type(4)));
        struct Loaded {
            ValuePair values[kSplit ? kUnroll / 2 : 1];
            uint32_t slots[kSplit ? kUnroll / 2 : 1];
            RecordWords whole[kSplit ? 1 : kUnroll];
        };
        // record u of a lane's kUnroll is record index_of(base, u) of the segment
        const auto index_of = [&](uint32_t base, uint32_t u) {
            return kSplit ? base + ((u >> 1) * 64 + lane) * 2 + (u & 1) : base + u * 64 + lane;
        };
        struct Cursor {
            uint32_t k, base;  // segment (of this wave's n_segments), first record of the chunk
        };
        // (Past the last chunk the loads are issued all the same, from the wave's first segment: with loads
        // behind a branch the compiler cannot tell how many are on their way when the other chunk is added, and
        // makes the adds wait for all of them.)
        const auto fetch = [&](const Cursor& at, Loaded& got) {
            const bool any = at.k < n_segments;
            const uint32_t count = any ? count_of(at.k) : 0u;
            const size_t seg = first + (g0 + (any ? at.k : 0u) * kWaves) * bins.segment_capacity;
            if constexpr (kSplit) {
                const RecordValues* values = static_cast<const RecordValues*>(bins.records) + seg;  // 16-byte aligned:
                const uint16_t* slots = bins.slots + seg;                                         // segments are multiples of four records
#pragma unroll
                for (uint32_t u = 0; u < kUnroll; u += 2) {
                    const uint32_t i = index_of(at.base, u);
                    const uint32_t from = i < count ? i : 0u;  // even; an odd count's last pair reads one record of the segment's slack
                    got.values[u / 2] = __builtin_nontemporal_load(reinterpret_cast<const ValuePair*>(values + from));
                    got.slots[u / 2] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(slots + from));
                }
            } else {
                const BinRecord* recs = static_cast<const BinRecord*>(bins.records) + seg;
#pragma unroll
                for (uint32_t u = 0; u < kUnroll; ++u) {
                    const uint32_t i = index_of(at.base, u);
                    got.whole[u] = __builtin_nontemporal_load(reinterpret_cast<const RecordWords*>(recs + (i < count ? i : 0u)));
                }
            }
        };
        const auto add = [&](const Cursor& at, const Loaded& got) {
            const uint32_t count = count_of(at.k);
#pragma unroll
            for (uint32_t u = 0; u < kUnroll; ++u) {
                uint32_t cell;
                float a0, a1;
                if constexpr (kSplit) {
                    const ValuePair v = got.values[u / 2];
                    const float v0 = v.x, v1 = v.y, v2 = v.z, v3 = v.w;  // copies first: a bit cast applied directly to a vector element reads element 0
                    cell = (u & 1) ? got.slots[u / 2] >> 16 : got.slots[u / 2] & 0xFFFFu;
                    a0 = (u & 1) ? v2 : v0;
                    a1 = (u & 1) ? v3 : v1;
                } else {
                    const RecordWords w = got.whole[u];
                    const uint32_t w0 = w.x, w1 = w.y, w2 = w.z;
                    cell = w0;
                    a0 = __builtin_bit_cast(float, w1);
                    a1 = __builtin_bit_cast(float, w2);
                }
                if (index_of(at.base, u) < count) {
                    __hip_atomic_fetch_add(&acc0[cell], static_cast<double>(a0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    __hip_atomic_fetch_add(&acc1[cell], static_cast<double>(a1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                }
            }
        };
        // the chunk after `at`: the next kChunk records of its segment, or the start of the next segment that has any
        const auto after = [&](Cursor at) {
            at.base += kChunk;
            if (at.base >= count_of(at.k)) {
                at.base = 0;
                do ++at.k; while (at.k < n_segments && count_of(at.k) == 0u);
            }
            return at;
        };
        // two sets of registers take turns, so a chunk's loads stay in flight over the other chunk's adds
        Cursor a{0u, 0u};
        while (a.k < n_segments && count_of(a.k) == 0u) ++a.k;
        Loaded got_a, got_b;
        if (a.k < n_segments) fetch(a, got_a);
        while (a.k < n_segments) {
            const Cursor b = after(a);
            fetch(b, got_b);
            add(a, got_a);
            if (b.k >= n_segments) break;
            a = after(b);
            fetch(a, got_a);
            add(b, got_b);
        }
    }
    // nothing has been added to the bin's slots since the gradient was cleared (or, for a caller who keeps the gradient
    // across calls, since that caller last cleared this slot range): the sums are the result.  Read before the barrier:
    // thread 0 sets the flag at the end.
    const bool untouched_so_far = bins.direct[bin] == 0u;
    __syncthreads();
    const GradSlice level_grad{table_grad + (static_cast<size_t>(level) * capacity * feat_pairs + pair) * 2, 2 * feat_pairs, nullptr, 0u};
    const uint32_t slot0 = bin << kBinSlotsLog2;  // (this kernel serves bins of kBinSlots slots only)
    const bool alone = gridDim.z == 1;
    if (alone) {
        // all of a thread's read-modify-writes at once: the loads are issued together, not one per trip
        constexpr int kMine = kBinSlots / kReduceBlock;
        float2 sum[kMine], g[kMine];
        bool touched[kMine];
#pragma unroll
        for (int k = 0; k < kMine; ++k) {
            const uint32_t s = static_cast<uint32_t>(k) * kReduceBlock + threadIdx.x;
            const double v0 = acc0[s], v1 = acc1[s];
            sum[k] = make_float2(static_cast<float>(v0), static_cast<float>(v1));
            touched[k] = (v0 != 0.0 || v1 != 0.0) && slot0 + s < capacity;
        }
#pragma unroll
        for (int k = 0; k < kMine; ++k) {
            const uint32_t s = static_cast<uint32_t>(k) * kReduceBlock + threadIdx.x;
            g[k] = make_float2(0.0f, 0.0f);
            if (touched[k] && !untouched_so_far) g[k] = *reinterpret_cast<const float2*>(level_grad.at(slot0 + s));
        }
#pragma unroll
        for (int k = 0; k < kMine; ++k) {
            const uint32_t s = static_cast<uint32_t>(k) * kReduceBlock + threadIdx.x;
            if (touched[k]) {
                g[k].x += sum[k].x;
                g[k].y += sum[k].y;
                *reinterpret_cast<float2*>(level_grad.at(slot0 + s)) = g[k];
            }
        }
        if (threadIdx.x == 0 && untouched_so_far) bins.direct[bin] = 1u;  // this slot range now holds sums
        return;
    }
    if (threadIdx.x == 0 && untouched_so_far) bins.direct[bin] = 1u;  // (the workgroups that share the bin all store the same value)
    for (uint32_t s = threadIdx.x; s < static_cast<uint32_t>(kBinSlots); s += kReduceBlock) {
        const double v0 = acc0[s], v1 = acc1[s];
        if ((v0 != 0.0 || v1 != 0.0) && slot0 + s < capacity) {
            float2* cell = reinterpret_cast<float2*>(level_grad.at(slot0 + s));
            global_add(&cell->x, static_cast<float>(v0));
            global_add(&cell->y, static_cast<float>(v1));
        }
    }
}

// A barrier that orders the workgroup's LDS accesses only.  __syncthreads() also makes the global stores
// issued so far visible, i.e. waits for the counter that loads share with them: after a store, it
// would wait for every load that is still on its way.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// The reducer of tables with hundreds of bins.  There a scattering workgroup leaves only a few
// dozen records in each of its segments and a (bin, level) has a few thousand in all, so a workgroup of
// bin_reduce_kernel is a chain of latencies (launch, counts, records, gradient) with nothing to overlap
// them: its 128 KiB of sums allow one workgroup per compute unit.  Here a workgroup keeps its bin and walks
// several levels (blockIdx.y, + gridDim.y, ...): the counts of all its levels are fetched at once
// (levels that left no records cost nothing more), and over the sequence of (level, 64 segments)
// steps that remain the counts are fetched two steps and the records one step ahead of the adds, so the
// loads of the next level are in flight while this level's sums are added and written out
// (measured on a 2^22-slot table, 16 levels, per call: bin_reduce_kernel 0.207 ms; this kernel 0.170 ms;
// with every load issued unconditionally, LDS-only barriers and a store-only write-out, so that nothing
// waits for the loads of the next step, 0.157 ms; with one workgroup per bin instead of two 0.146 ms).
// A quarter of a wave reads a segment, kLevelsShortUnroll records per lane: needs segments of at
// most kLevelsMaxSegment records, whole (12-byte) records, at most kReduceBlock groups and
// at most kLevelsMaxPerWorkgroup levels per workgroup (the host checks all four).
constexpr uint32_t kLevelsShortLanes = 16, kLevelsShortUnroll = 8;
constexpr uint32_t kLevelsMaxSegment = kLevelsShortLanes * kLevelsShortUnroll;
constexpr uint32_t kLevelsMaxPerWorkgroup = 24;
__global__ void __launch_bounds__(kReduceBlock)
bin_reduce_levels_kernel(BinTarget pass_bins, const float* __restrict__ window, uint32_t capacity, uint32_t feat_pairs,
                         float* __restrict__ table_grad, int first_level, uint32_t n_levels_in_pass) {
    __shared__ double acc0[kBinSlots];
    __shared__ double acc1[kBinSlots];
    __shared__ uint32_t masks[2];  // bit i: the workgroup's i-th level [0] has records in this bin, [1] got direct adds in this bin's slots
    const uint32_t bin = blockIdx.x, my_first = blockIdx.y, my_stride = gridDim.y;
    const uint32_t n_mine = (n_levels_in_pass - my_first + my_stride - 1) / my_stride;  // blockIdx.y < n_levels_in_pass
    const uint32_t n_bins = pass_bins.n_bins, n_groups = pass_bins.n_groups, seg_cap = pass_bins.segment_capacity;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // the workgroup's i-th level within the pass, and where its segments of this bin start (counted in segments)
    const auto level_in_pass = [&](uint32_t i) { return my_first + i * my_stride; };
    const auto first_segment = [&](uint32_t i) { return (static_cast<size_t>(level_in_pass(i)) * n_bins + bin) * n_groups; };
    if (threadIdx.x < 2) masks[threadIdx.x] = 0u;
    for (int s = threadIdx.x; s < kBinSlots; s += kReduceBlock) {
        acc0[s] = 0.0;
        acc1[s] = 0.0;
    }
    // which of the levels have records here (thread g looks at group g's count of every level, all loads at once)
    uint32_t seen[kLevelsMaxPerWorkgroup];
#pragma unroll
    for (uint32_t i = 0; i < kLevelsMaxPerWorkgroup; ++i) {
        seen[i] = 0u;
        if (i < n_mine) {
            const uint32_t pair_level = static_cast<uint32_t>(first_level) + level_in_pass(i);
            // (a masked level's scattering workgroups wrote no counts)
            if (window[pair_level / feat_pairs] != 0.0f && threadIdx.x < n_groups) seen[i] = pass_bins.counts[first_segment(i) + threadIdx.x];
        }
    }
    uint32_t direct = 0u;
    if (threadIdx.x < n_mine) direct = pass_bins.direct[static_cast<size_t>(level_in_pass(threadIdx.x)) * n_bins + bin];
    __syncthreads();  // the masks are cleared
    uint32_t found = 0u;
#pragma unroll
    for (uint32_t i = 0; i < kLevelsMaxPerWorkgroup; ++i)
        if (__ballot(seen[i] != 0u) != 0ull) found |= 1u << i;
    if (lane == 0 && found != 0u) atomicOr(&masks[0], found);
    if (direct != 0u) atomicOr(&masks[1], 1u << threadIdx.x);
    __syncthreads();
    const uint32_t todo = masks[0], direct_mask = masks[1];
    if (todo == 0u) return;

    // a step: 64 segments of one level, one per quarter wave
    constexpr uint32_t kEnd = 32;
    // Bins wider than the LDS sums (tables above 2^22 slots) are summed one range of kBinSlots slots after
    // the other: every range walks all the bin's records and takes those that fall into it.
    const uint32_t n_ranges = 1u << (pass_bins.bin_shift - kBinSlotsLog2);
    struct Cursor {
        uint32_t i, range, step;  // the workgroup's i-th level (kEnd: past the last), the range of the bin, segments 64 * step ...
    };
    const uint32_t n_steps = (n_groups + 63) / 64;
    const auto after = [&](Cursor at) {
        if (++at.step < n_steps) return at;
        at.step = 0u;
        if (++at.range < n_ranges) return at;
        const uint32_t rest = at.i + 1 < 32 ? todo >> (at.i + 1) : 0u;
        return Cursor{rest != 0u ? at.i + 1 + static_cast<uint32_t>(__builtin_ctz(rest)) : kEnd, 0u, 0u};
    };
    const uint32_t reader = wave * 4 + lane / kLevelsShortLanes, l = lane % kLevelsShortLanes;
    // (Every load below is issued whether or not its result is wanted, from an address that is valid
    // either way: with loads behind branches the compiler cannot tell how many are on their way and
    // makes every use wait for all of them, those of the next step included.)
    const auto load_count = [&](const Cursor& at) {
        const uint32_t g = at.step * 64 + reader;
        const uint32_t i = at.i != kEnd ? at.i : 0u;
        const uint32_t count = pass_bins.counts[first_segment(i) + (g < n_groups ? g : 0u)];
        return at.i != kEnd && g < n_groups ? count : 0u;
    };
    struct Loaded {
        RecordWords rec[kLevelsShortUnroll];
        uint32_t count, range;
    };
    const BinRecord* const records = static_cast<const BinRecord*>(pass_bins.records);
    const auto fetch = [&](const Cursor& at, uint32_t count, Loaded& got) {
        const uint32_t g = at.step * 64 + reader;
        const BinRecord* seg = records + (first_segment(at.i != kEnd ? at.i : 0u) + (g < n_groups ? g : 0u)) * seg_cap;
        got.count = count;
        got.range = at.range;
#pragma unroll
        for (uint32_t u = 0; u < kLevelsShortUnroll; ++u) {
            const uint32_t idx = u * kLevelsShortLanes + l;
            // (normal loads: neighbouring short segments share cache lines); the pass's first record stands in where there is none
            got.rec[u] = *reinterpret_cast<const RecordWords*>(idx < count ? seg + idx : records);
        }
    };
    const auto add = [&](const Loaded& got) {
#pragma unroll
        for (uint32_t u = 0; u < kLevelsShortUnroll; ++u) {
            const RecordWords w = got.rec[u];
            const uint32_t w0 = w.x, w1 = w.y, w2 = w.z;  // copies first: a bit cast applied directly to a vector element reads element 0
            if (u * kLevelsShortLanes + l < got.count && (w0 >> kBinSlotsLog2) == got.range) {
                const uint32_t cell = w0 & (kBinSlots - 1);
                __hip_atomic_fetch_add(&acc0[cell], static_cast<double>(__builtin_bit_cast(float, w1)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_fetch_add(&acc1[cell], static_cast<double>(__builtin_bit_cast(float, w2)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
    };
    // Adds the sums of one range of the bin at the workgroup's i-th level into the gradient and clears them.  Nothing else touches
    // the bin's slots of that level while this kernel runs, so the add is a plain read-modify-write, or a
    // store where nothing was added since the gradient was cleared.
    const auto flush = [&](uint32_t i, uint32_t range) {
        lds_barrier();
        const uint32_t pair_level = static_cast<uint32_t>(first_level) + level_in_pass(i);
        const uint32_t level = pair_level / feat_pairs, pair = pair_level % feat_pairs;
        const GradSlice level_grad{table_grad + (static_cast<size_t>(level) * capacity * feat_pairs + pair) * 2, 2 * feat_pairs, nullptr, 0u};
        const uint32_t slot0 = (bin << pass_bins.bin_shift) + (range << kBinSlotsLog2);
        const bool untouched_so_far = ((direct_mask >> i) & 1u) == 0u;
        if (threadIdx.x == 0 && untouched_so_far) pass_bins.direct[static_cast<size_t>(level_in_pass(i)) * n_bins + bin] = 1u;  // this slot range now holds sums
        constexpr int kMine = kBinSlots / kReduceBlock;
        // (two loops, so that the usual one has no load to wait for: a wait would also be one for the
        // records of the next step, which are on their way)
        if (untouched_so_far) {
#pragma unroll
            for (int k = 0; k < kMine; ++k) {
                const uint32_t s = static_cast<uint32_t>(k) * kReduceBlock + threadIdx.x;
                const double v0 = acc0[s], v1 = acc1[s];
                if (v0 != 0.0 || v1 != 0.0) {
                    acc0[s] = 0.0;
                    acc1[s] = 0.0;
                    if (slot0 + s < capacity)
                        *reinterpret_cast<float2*>(level_grad.at(slot0 + s)) = make_float2(static_cast<float>(v0), static_cast<float>(v1));
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < kMine; ++k) {
                const uint32_t s = static_cast<uint32_t>(k) * kReduceBlock + threadIdx.x;
                const double v0 = acc0[s], v1 = acc1[s];
                if (v0 != 0.0 || v1 != 0.0) {
                    acc0[s] = 0.0;
                    acc1[s] = 0.0;
                    if (slot0 + s < capacity) {
                        float2* cell = reinterpret_cast<float2*>(level_grad.at(slot0 + s));
                        float2 g = *cell;
                        g.x += static_cast<float>(v0);
                        g.y += static_cast<float>(v1);
                        *cell = g;
                    }
                }
            }
        }
        lds_barrier();
    };
    // two sets of registers take turns for the records, two registers for the counts; past the last step the
    // counts are zero and the loads fetch the stand-in
    Cursor it0{static_cast<uint32_t>(__builtin_ctz(todo)), 0u, 0u};
    Cursor it1 = after(it0);
    uint32_t count_x = load_count(it0), count_y = load_count(it1);
    Loaded got_a, got_b;
    fetch(it0, count_x, got_a);
    while (true) {
        const Cursor it2 = it1.i != kEnd ? after(it1) : it1;
        count_x = load_count(it2);
        fetch(it1, count_y, got_b);
        add(got_a);
        if (it1.i != it0.i || it1.range != it0.range) flush(it0.i, it0.range);
        if (it1.i == kEnd) break;
        const Cursor it3 = it2.i != kEnd ? after(it2) : it2;
        count_y = load_count(it3);
        fetch(it2, count_x, got_a);
        add(got_b);
        if (it2.i != it1.i || it2.range != it1.range) flush(it1.i, it1.range);
        if (it2.i == kEnd) break;
        it0 = it2;
        it1 = it3;
    }
}

}  // namespace penc
