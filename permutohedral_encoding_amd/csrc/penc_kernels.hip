// HIP kernels (gfx950, wave64) and C-ABI entry points of the permutohedral-lattice hash encoding.
//
// Work decomposition (one thread per (point, level) everywhere)
//   forward, grad-of-grad (the gathering half of the double backward) : blockIdx.y is the level, so
//       consecutive workgroups work on the same 8*capacity-byte slice of the table, which stays in
//       L2, and the level's scale factors / shifts / window weight are wave-uniform (scalar loads).
//   position backward : a thread sums a group of two levels in registers; the per-group partial
//       sums are reduced in a fixed order, without atomics (the reference needs D atomics per
//       point-level because it gives each level its own block,
//       kernels/permutohedral_encoding/EncodingGPU.cuh:745-750).
//   table backward (first order and the scattering half of the double backward) : workgroups of
//       512 threads walk groups of 8 or 16 tiles of points; neighbouring workgroups of a die take
//       the same points at different levels.  The scatter itself (LDS accumulate cache, slot-range
//       bins, direct atomics) is described in penc_scatter.hpp.
//   A level whose anneal-window weight is exactly 0 contributes exactly 0 everywhere (for finite
//   table values), so such levels skip the table traffic and only store their zeros.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>
#include <type_traits>

#include "../../include/penc.h"
#include "penc_lattice.hpp"
#include "penc_scatter.hpp"

namespace penc {

// Levels one position-gradient thread sums in registers (measured: 2 is fastest up to D = 5, 1
// from D = 6 on, where a thread's arithmetic per level is long enough; 3 and 4 are slower everywhere,
// also with all their gathers issued up front: more levels at a time overflow L2).
constexpr int pos_levels_per_group(int pos_dim) { return pos_dim >= 6 ? 1 : 2; }

constexpr int kDefaultLevelsPerPass = 1 << 20;  // by default the suggested workspace bins all levels in one pass (measured fastest)

template <int D>
__device__ __forceinline__ fvec<D> load_point(const float* __restrict__ positions, int64_t n) {
    const float* p = positions + n * D;
    fvec<D> pos;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i); pos[i] = p[i]; });
    return pos;
}

// The D+1 table entries of a simplex (F features each: one load of F elements per vertex, two of 16
// bytes for eight floats), fetched back to back so that all loads are in flight together.
// f[k][r] is feature k of vertex r.  T is the table's element type: float, or __half / bfloat16_bits
// for a table kept in 16 bits (the values are widened exactly; all arithmetic stays fp32).
struct bfloat16_bits {
    uint16_t bits;  // the upper half of the fp32 with the same value
};
template <int D, int F>
struct Vertices {
    fvec<D + 1> f[F];
};
template <int D, int F, typename T>
__device__ __forceinline__ Vertices<D, F> load_vertices(const T* __restrict__ level_table, uvec<D + 1> h,
                                                        uint32_t capacity, uint32_t cap_mask) {
    static_assert(F == 2 || F == 4 || F == 8, "two, four or eight features per level");
    Vertices<D, F> v;
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        const size_t slot = to_slot(h[r], capacity, cap_mask);
        if constexpr (sizeof(T) == 2) {
            // F halves in one load of 4, 8 or 16 bytes
            using Packed = typename std::conditional<F == 2, uint32_t, typename std::conditional<F == 4, uint2, uint4>::type>::type;
            const Packed raw = *reinterpret_cast<const Packed*>(level_table + F * slot);
            uint32_t words[F / 2];
            __builtin_memcpy(words, &raw, sizeof(raw));
            static_for<F / 2>(PENC_BODY(q) {
                PENC_INDEX(q);
                if constexpr (std::is_same<T, bfloat16_bits>::value) {
                    v.f[2 * q + 0][r] = __builtin_bit_cast(float, words[q] << 16);
                    v.f[2 * q + 1][r] = __builtin_bit_cast(float, words[q] & 0xFFFF0000u);
                } else {
                    const float2 x = __half22float2(__builtin_bit_cast(__half2, words[q]));
                    v.f[2 * q + 0][r] = x.x;
                    v.f[2 * q + 1][r] = x.y;
                }
            });
        } else if constexpr (F == 2) {
            const float2 x = *reinterpret_cast<const float2*>(level_table + 2 * slot);
            v.f[0][r] = x.x;
            v.f[1][r] = x.y;
        } else {
            static_for<F / 4>(PENC_BODY(q) {
                PENC_INDEX(q);
                const float4 x = *reinterpret_cast<const float4*>(level_table + F * slot + 4 * q);
                v.f[4 * q + 0][r] = x.x;
                v.f[4 * q + 1][r] = x.y;
                v.f[4 * q + 2][r] = x.z;
                v.f[4 * q + 3][r] = x.w;
            });
        }
    });
    return v;
}

// ------------------------------------------------------------------------------------------
// forward (EncodingGPU.cuh:68-256)
//
// One thread per point and one or two levels (the host says which).  Measured alternatives, all
// slower or equal: 2 or 4 points per
// thread (more loads in flight per lane: no gain, the kernel already runs at the rate this GPU
// sustains for random 8-byte loads from a 2 MiB slice); walking all the levels inside the thread with
// the positions kept in registers (20% slower at 2^20 points, 3x slower at 2^16: fewer, longer
// waves lose more than the re-read positions cost); interleaving workgroups of a coarse
// (compute-bound) and a fine (gather-bound) level, which takes the fine level's slice out of L2
// (30% slower).

template <int D, int F, typename T>
__global__ void __launch_bounds__(kBlock)
forward_kernel(int n_points, int n_levels, int n_all_levels, int levels_per_thread, uint32_t capacity, uint32_t cap_mask,
               const float* __restrict__ positions, const T* __restrict__ table,
               const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
               const float* __restrict__ window, float* __restrict__ sliced, float points_scaling) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    __shared__ uint2 columns[(D + 1) * kBlock];
    const fvec<D> point = load_point<D>(positions, n);
    // The levels of a thread are `gridDim.y` apart: with the usual coarse-to-fine level list a thread that
    // takes two pairs a level whose gathers hit the first-level cache with one that waits for the L2.
#pragma unroll 1
    for (int k2 = 0; k2 < levels_per_thread; ++k2) {
        const int level = static_cast<int>(blockIdx.y) + k2 * static_cast<int>(gridDim.y);
        if (level >= n_all_levels) break;
        float* out = sliced + (static_cast<size_t>(level) * F) * n_points + n;  // feature k at out[k * n_points]

        if (level >= n_levels) {  // extra levels carrying the raw positions (:106-121)
            const int src = (level - n_levels) * F;
            const float* p = positions + static_cast<size_t>(n) * D;
            static_for<F>(PENC_BODY(k) {
                PENC_INDEX(k);
                out[static_cast<size_t>(k) * n_points] = src + k < D ? p[src + k] * points_scaling : 0.0f;
            });
            continue;
        }
        const float w_level = window[level];
        if (w_level == 0.0f) {
            static_for<F>(PENC_BODY(k) {
                PENC_INDEX(k); out[static_cast<size_t>(k) * n_points] = 0.0f; });
            continue;
        }
        const Located<D> s = locate<D>(point, random_shift + level * D, scale_factor + level * D);
        // residuals and hash steps into rank order through LDS: up to 6% faster than the select chains
        // of vertex_hashes() / barycentric() at D = 8, equal at D = 3
        uvec<D + 1> h;
        fvec<D + 1> sorted;
        sort_by_rank_lds<D>(columns + threadIdx.x, kBlock, s.rank, s.delta, s.hash0, sorted, h);
        const fvec<D + 1> w = barycentric_of_sorted<D>(sorted);
        const Vertices<D, F> v = load_vertices<D, F, T>(table + static_cast<size_t>(level) * capacity * F, h, capacity, cap_mask);
        fvec<F> acc = 0.0f;
        static_for<D + 1>(PENC_BODY(r) {
            PENC_INDEX(r);
            const float wr = w[r] * w_level;
            static_for<F>(PENC_BODY(k) {
                PENC_INDEX(k); acc[k] = acc[k] + v.f[k][r] * wr; });
        });
        static_for<F>(PENC_BODY(k) {
            PENC_INDEX(k);
            // written once and not read here: the non-temporal hint keeps it from displacing the level's table slice
            __builtin_nontemporal_store(acc[k], out + static_cast<size_t>(k) * n_points);
        });
    }
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. the table (EncodingGPU.cuh:259-414)

// Wavefronts per SIMD the scattering kernel is compiled for: six (three workgroups per compute unit, at
// most 80 vector registers) where that costs a few spilled registers at most, else four (two
// workgroups, 128 registers).  Measured at 2^19 points, 24 levels: table backward 0.367 -> 0.338 ms
// at D = 4 (84 -> 80 registers, 3 spilled), 0.458 -> 0.424 ms at D = 5; the second-order kernel
// 0.577 -> 0.552 ms at D = 4, but 0.735 -> 0.754 ms at D = 5 (11 spilled), which therefore stays at
// four; at D = 8 the second-order kernel needed 130 registers and ran one workgroup per compute
// unit: held to 128, 1.334 -> 1.113 ms.
constexpr int scatter_waves_per_simd(int pos_dim, bool second_order, bool wide_bins) {
    if (wide_bins) return pos_dim <= 3 ? 6 : 4;  // (a variable bin width takes six to eight more registers: up to 30 spilled at D = 4)
    return pos_dim <= 4 || (pos_dim == 5 && !second_order) ? 6 : 4;
}

// kRowMajor: the upstream gradient is read as rows grad[n][2*level + feature] of `grad_row_stride`
// floats (what the layer after the encoding produces) instead of [level][feature][n].  A die walks
// all levels of a group of points back to back, so the rows mostly come from L2 (measured: fetched
// from memory 2.7 times, not once per level) although every level only uses 8 bytes of each.
// With `grad_level_major` the kernel also leaves the values it read in [level][feature][n] order
// (for the position-gradient kernel, which gathers level by level and wants its upstream gradient
// coalesced): the layout change rides on reads this kernel makes anyway.
// kSecondOrder: the table-gradient half of the double backward (EncodingGPU.cuh:1016-1257): the
// vertex weights are the derivatives of the barycentric weights along `double_pos_grad` instead of
// the barycentric weights themselves; everything else is the same scatter.
// feat_pairs: with four or eight features per level the pairs (0,1), (2,3), ... are scattered like levels that
// share their geometry: "levels" below (first_level, n_pass_levels, the grid, the bins) count pairs,
// `pair_level` = level * feat_pairs + pair.  The upstream gradient needs no special case: [L][F][N]
// is [L * F/2][2][N], and in a row the pair sits at column 2 * pair_level.
// kWideBins: the bins span more than kBinSlots slots (tables above 2^22 slots).  A parameter of the kernel
// rather than a value read from its arguments, because with the bin width a variable the usual instances
// need up to eight more vector registers (at D = 4, held to 80 registers, 27 spilled instead of 5).
template <int D, bool kRowMajor, bool kSecondOrder, bool kWideBins>
__global__ void __launch_bounds__(kScatterBlock, scatter_waves_per_simd(D, kSecondOrder, kWideBins))
backward_table_kernel(int n_points, int first_level, uint32_t n_pass_levels, uint32_t feat_pairs, uint32_t dies, int tiles_per_group,
                      uint32_t capacity, uint32_t cap_mask,
                      const float* __restrict__ positions, const float* __restrict__ scale_factor,
                      const float* __restrict__ random_shift, const float* __restrict__ window,
                      const float* __restrict__ grad_sliced, int64_t grad_row_stride,
                      const float* __restrict__ double_pos_grad, float* __restrict__ table_grad,
                      float* __restrict__ grad_level_major, BinTarget pass_bins) {
    __shared__ ScatterStateT<stage_chunk(D)> state;
    // Workgroups are dealt round-robin to the chip's `dies` dies, each with an L2 of its own.  The j-th
    // workgroup of a die takes level j % levels of one group of points: a die works through all
    // levels of a group before the next group, so the points are fetched from memory once, and
    // compute-bound coarse levels and store-bound fine levels share the chip at all times (this
    // kernel never reads the table: there is no slice to keep cache-resident by running a level at
    // a time).
    const uint32_t die = blockIdx.x % dies, j = blockIdx.x / dies;
    const uint32_t level_in_pass = j % n_pass_levels, group = (j / n_pass_levels) * dies + die;
    const int64_t group_base = static_cast<int64_t>(group) * tiles_per_group * kScatterBlock;
    if (group_base >= n_points) return;
    const uint32_t pair_level = static_cast<uint32_t>(first_level) + level_in_pass;
    const int level = static_cast<int>(pair_level / feat_pairs);  // the geometry's level
    const float w_level = window[level];
    if (w_level == 0.0f) return;
    scatter_begin(state);
    BinTarget bins = bins_of_level(pass_bins, level_in_pass);
    if constexpr (!kWideBins) bins.bin_shift = kBinSlotsLog2;  // a constant from here on
    const GradSlice level_grad{table_grad + (static_cast<size_t>(level) * capacity * feat_pairs + pair_level % feat_pairs) * 2,
                               2 * feat_pairs, bins.direct, bins.bin_shift};
    // Everything a thread reads lies within its group of at most 16 x 512 points, so the addresses are
    // wave-uniform 64-bit bases (scalar registers) plus 32-bit per-thread offsets.
    const uint32_t last_in_group = static_cast<uint32_t>(n_points - 1 - group_base);
    const float* const group_positions = positions + group_base * D;
    const float* const group_q = kSecondOrder ? double_pos_grad + group_base * D : nullptr;
    const float* const group_grad0 =
        kRowMajor ? grad_sliced + group_base * grad_row_stride + 2 * pair_level
                  : grad_sliced + (static_cast<size_t>(pair_level) * 2) * n_points + group_base;
    const float* const group_grad1 = group_grad0 + n_points;
    const auto load_grad = [&](uint32_t i, float& g0, float& g1) {
        if constexpr (kRowMajor) {
            const float2 g = *reinterpret_cast<const float2*>(group_grad0 + static_cast<int64_t>(i) * grad_row_stride);
            g0 = g.x;
            g1 = g.y;
        } else {
            g0 = group_grad0[i];
            g1 = group_grad1[i];
        }
    };
    const auto load_group_point = [&](const float* base, uint32_t i) {
        fvec<D> v;
        static_for<D>(PENC_BODY(k) {
            PENC_INDEX(k); v[k] = base[i * static_cast<uint32_t>(D) + k]; });
        return v;
    };
    // A tile's inputs are fetched one tile ahead: their latency then overlaps the previous tile's
    // scatter instead of stalling the wave at the top of every iteration.
    const auto point_of = [&](int t) {  // the point this thread handles in tile t, within the group (clamped: the tail re-reads the last point)
        const uint32_t i = static_cast<uint32_t>(t) * kScatterBlock + threadIdx.x;
        return i < last_in_group ? i : last_in_group;
    };
    uint32_t nn = point_of(0);
    fvec<D> pos = load_group_point(group_positions, nn);
    fvec<D> q = 0.0f;
    if constexpr (kSecondOrder) q = load_group_point(group_q, nn);
    float g0, g1;
    load_grad(nn, g0, g1);
    int mode = kModeCache;
    uint32_t id_bits = 0;
    for (int t = 0; t < tiles_per_group; ++t) {
        const int64_t tile_base = group_base + static_cast<int64_t>(t) * kScatterBlock;
        if (tile_base >= n_points) break;
        const bool active = tile_base + threadIdx.x < n_points;
        const uint32_t nn_next = point_of(t + 1);
        const fvec<D> pos_next = load_group_point(group_positions, nn_next);
        fvec<D> q_next = 0.0f;
        if constexpr (kSecondOrder) q_next = load_group_point(group_q, nn_next);
        float g0_next, g1_next;
        load_grad(nn_next, g0_next, g1_next);
        if constexpr (kRowMajor) {
            if (grad_level_major != nullptr && active) {
                float* out = grad_level_major + (static_cast<size_t>(pair_level) * 2) * n_points + tile_base + threadIdx.x;
                out[0] = g0;
                out[n_points] = g1;
            }
        }
        const Located<D> s = locate<D>(pos, random_shift + level * D, scale_factor + level * D);
        uvec<D + 1> h;
        fvec<D + 1> w;  // b_r * w_level (:405), or dB[r] * w_level (:1244-1245)
        bool via_lds = false;
        if constexpr (D > kWorkgroupSortMaxDim) {
            // Once the workgroup streams with every wave sorting on its own (stream_tile_wave), a wave's staging
            // slice is idle between its tiles and nobody else touches it: it serves as the thread-private
            // columns that put residuals and hash steps into rank order, in place of D(D+1) selects each
            // (at D = 8 about 270 of 1350 vector instructions per point and level).
            via_lds = mode == kModeStream && bins.n_bins <= static_cast<uint32_t>(kStageBins);
        }
        if (via_lds) {
            constexpr uint32_t kSliceCells = ScatterStateT<stage_chunk(D)>::kChunk * 64 * 2;  // 8-byte cells of a wave's slice
            static_assert((D + 1) * 64 <= kSliceCells, "a wave's staging slice holds a column of D+1 cells per lane");
            uint2* const column = reinterpret_cast<uint2*>(state.val) + (threadIdx.x >> 6) * kSliceCells + (threadIdx.x & 63);
            fvec<D + 1> sorted;
            if constexpr (kSecondOrder) {
                sort_by_rank_lds<D>(column, 64, s.rank, pos_grad_grad_to_elevated<D>(q, scale_factor + level * D), s.hash0, sorted, h);
                w = sorted_elevated_grad_to_bary<D>(sorted) * w_level;
            } else {
                sort_by_rank_lds<D>(column, 64, s.rank, s.delta, s.hash0, sorted, h);
                w = barycentric_of_sorted<D>(sorted) * w_level;
            }
            wave_lds_fence();  // the slice is staging space again from here on
        } else {
            h = vertex_hashes<D>(s.rank, s.hash0);
            if constexpr (kSecondOrder) {
                w = pos_grad_grad_to_bary<D>(s.rank, q, scale_factor + level * D) * w_level;
            } else {
                w = barycentric<D>(s.rank, s.delta) * w_level;
            }
        }
        uvec<D + 1> slot;
        static_for<D + 1>(PENC_BODY(r) {
            PENC_INDEX(r);
            slot[r] = to_slot(h[r], capacity, cap_mask);
        });
        if (t == 0) {
            // the next tile's slots, should the decision want to know whether its points use the slots this tile uses
            // (its point is already here)
            const auto slots_of_next_tile = [&]() {
                const Located<D> s1 = locate<D>(pos_next, random_shift + level * D, scale_factor + level * D);
                const uvec<D + 1> h1 = vertex_hashes<D>(s1.rank, s1.hash0);
                uvec<D + 1> slot1;
                static_for<D + 1>(PENC_BODY(r) {
                    PENC_INDEX(r);
                    slot1[r] = to_slot(h1[r], capacity, cap_mask);
                });
                return slot1;
            };
            const bool next_active = tile_base + kScatterBlock + threadIdx.x < n_points && tiles_per_group > 1;
            mode = scatter_mode_decide<D>(state, bins, active, slot, id_bits, next_active, slots_of_next_tile, tiles_per_group);
        }
        const uint32_t hits = scatter_tile<D>(state, level_grad, bins, group, active, cache_pays<D>(state, t),
                                              mode, id_bits, slot, w * g0, w * g1);  // g_f * (b_r * w_level), :405-410
        // the first tile finds the lines its own look-up has claimed: no evidence of reuse
        if ((threadIdx.x & 63) == 0 && hits && t > 0) atomicAdd(&state.hits, hits);
        pos = pos_next;
        q = q_next;
        g0 = g0_next;
        g1 = g1_next;
    }
    scatter_end(state, level_grad, bins, group, mode, id_bits);
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. positions (EncodingGPU.cuh:530-769)

// One thread per (point, group of levels): the levels of the group are summed in
// registers and stored once, at out[group][point][D].  With a single group (no workspace) `out` is
// the position gradient itself; otherwise it is a partial buffer that reduce_level_groups_kernel
// sums, in ascending group order, so the result is deterministic either way.  Small groups keep
// the whole chip on the same few levels at a time (their table slices stay in L2) and give the
// launch many more, shorter waves than one thread per point walking all levels.  (Doing this
// kernel's rank permutations through LDS, as the forward does, was measured: no gain.)
template <int D, int F, typename T>
__global__ void __launch_bounds__(kBlock)
backward_pos_kernel(int n_points, int n_levels, int levels_per_group, uint32_t capacity, uint32_t cap_mask,
                    const float* __restrict__ positions, const T* __restrict__ table,
                    const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                    const float* __restrict__ window, const float* __restrict__ grad_sliced,
                    float* __restrict__ out) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    const fvec<D> pos = load_point<D>(positions, n);
    fvec<D> total = 0.0f;
    // The levels of a group are `gridDim.y` apart, not adjacent: with the usual coarse-to-fine level list a
    // group then pairs a coarse level, whose points share few slots, with a fine one, and the table slices
    // the whole chip gathers from at any time fit the L2 (two adjacent fine levels are 4 MiB at 2^18 slots,
    // an L2's whole capacity).
    for (int k = 0; k < levels_per_group; ++k) {
        const int level = static_cast<int>(blockIdx.y) + k * static_cast<int>(gridDim.y);
        if (level >= n_levels) break;
        const float w_level = window[level];
        if (w_level == 0.0f) continue;
        const float* sf = scale_factor + level * D;
        const Located<D> s = locate<D>(pos, random_shift + level * D, sf);
        const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
        const Vertices<D, F> v = load_vertices<D, F, T>(table + static_cast<size_t>(level) * capacity * F, h, capacity, cap_mask);
        const float* gp = grad_sliced + (static_cast<size_t>(level) * F) * n_points + n;
        // the upstream gradient is read once (non-temporal: it should not displace the table slices)
        fvec<D + 1> dB = (v.f[0] * w_level) * __builtin_nontemporal_load(gp);  // :688-689, feature by feature
        static_for<F - 1>(PENC_BODY(kk) {
            PENC_INDEX(kk);
            constexpr int k = kk + 1;
            dB += (v.f[k] * w_level) * __builtin_nontemporal_load(gp + static_cast<size_t>(k) * n_points);
        });
        total += bary_grad_to_pos_grad<D>(s.rank, dB, sf);
    }
    float* o = out + (static_cast<size_t>(blockIdx.y) * n_points + n) * D;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i);
        o[i] = total[i];
    });
}

__global__ void __launch_bounds__(kBlock)
reduce_level_groups_kernel(const float* __restrict__ partial, int n_groups, size_t n_values, float* __restrict__ out) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n_values; i += stride) {
        float acc = partial[i];
        for (int g = 1; g < n_groups; ++g) acc += partial[static_cast<size_t>(g) * n_values + i];
        out[i] = acc;
    }
}

// ------------------------------------------------------------------------------------------
// double backward from d(loss)/d(position gradient), the half that gathers: gradient w.r.t.
// grad_sliced_values (EncodingGPU.cuh:1260-1493).  One thread per (point, level), a level at a
// time, like the forward.  (The other half, the scatter into the table gradient, is
// backward_table_kernel<D, false, true>.  One kernel doing both, with eight tiles per workgroup,
// was measured 7-13% slower than the two: the gathering half wants small workgroups, the scattering
// half large groups of points with the levels interleaved.)

template <int D, int F, typename T>
__global__ void __launch_bounds__(kBlock)
grad_grad_kernel(int n_points, int n_levels, int n_all_levels, int levels_per_thread, uint32_t capacity, uint32_t cap_mask,
                 const float* __restrict__ positions, const T* __restrict__ table,
                 const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                 const float* __restrict__ window, const float* __restrict__ double_pos_grad,
                 float* __restrict__ grad_grad_sliced) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    __shared__ uint2 columns[(D + 1) * kBlock];
    const fvec<D> point = load_point<D>(positions, n), q = load_point<D>(double_pos_grad, n);
    // the levels of a thread are `gridDim.y` apart, as in the forward
#pragma unroll 1
    for (int k2 = 0; k2 < levels_per_thread; ++k2) {
        const int level = static_cast<int>(blockIdx.y) + k2 * static_cast<int>(gridDim.y);
        if (level >= n_all_levels) break;
        float* o = grad_grad_sliced + (static_cast<size_t>(level) * F) * n_points + n;
        const float w_level = level < n_levels ? window[level] : 0.0f;  // concat levels: zeros (:1290-1295)
        if (w_level == 0.0f) {
            static_for<F>(PENC_BODY(k) {
                PENC_INDEX(k); o[static_cast<size_t>(k) * n_points] = 0.0f; });
            continue;
        }
        const float* sf = scale_factor + level * D;
        const Located<D> s = locate<D>(point, random_shift + level * D, sf);
        // one trip through the thread's LDS column puts both the elevated gradient and the hash steps
        // into rank order (as in the forward)
        uvec<D + 1> h;
        fvec<D + 1> sorted;
        sort_by_rank_lds<D>(columns + threadIdx.x, kBlock, s.rank, pos_grad_grad_to_elevated<D>(q, sf), s.hash0, sorted, h);
        const Vertices<D, F> v = load_vertices<D, F, T>(table + static_cast<size_t>(level) * capacity * F, h, capacity, cap_mask);
        // dB[r] * w_level, then times the vertex value (:1484-1485)
        const fvec<D + 1> wr = sorted_elevated_grad_to_bary<D>(sorted) * w_level;
        fvec<F> gg = 0.0f;
        static_for<D + 1>(PENC_BODY(r) {
            PENC_INDEX(r);
            static_for<F>(PENC_BODY(k) {
                PENC_INDEX(k); gg[k] += wr[r] * v.f[k][r]; });
        });
        static_for<F>(PENC_BODY(k) {
            PENC_INDEX(k); o[static_cast<size_t>(k) * n_points] = gg[k]; });
    }
}

// ------------------------------------------------------------------------------------------
// optimiser step on the table

// One fused AdamW update (decoupled weight decay, no amsgrad) in the order torch.optim.AdamW applies
// it: p *= 1 - lr*wd; m += (1-b1)(g - m); v = b2 v + (1-b2) g^2; p -= step_size * m / (sqrt(v)/c2 + eps).
// With skip_zero an entry whose gradient is exactly 0 is left alone altogether (moments, decay and
// value), which is how hash-grid tables are usually trained: most slots of a large table get no
// gradient in a step.  Four values per thread where the arrays allow 16-byte accesses.
struct AdamWStep {
    float decay;        // 1 - lr * weight_decay
    float one_minus_b1, b2, one_minus_b2;
    float step_size;    // lr / (1 - b1^step)
    float inv_c2;       // 1 / sqrt(1 - b2^step)
    float eps;
};
__device__ __forceinline__ void adamw_update(const AdamWStep& a, bool skip_zero, float g, float& p, float& m, float& v) {
    if (skip_zero && g == 0.0f) return;
    p = p * a.decay;
    m = m + a.one_minus_b1 * (g - m);
    v = v * a.b2 + a.one_minus_b2 * (g * g);
    p = p - a.step_size * (m / (__builtin_sqrtf(v) * a.inv_c2 + a.eps));
}
template <bool kVector>
__global__ void __launch_bounds__(kBlock)
adamw_step_kernel(float* __restrict__ params, const float* __restrict__ grads, float* __restrict__ exp_avg,
                  float* __restrict__ exp_avg_sq, size_t n, AdamWStep a, int skip_zero) {
    const size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if constexpr (kVector) {
        if (i * 4 >= n) return;
        const float4 g = reinterpret_cast<const float4*>(grads)[i];
        if (skip_zero && g.x == 0.0f && g.y == 0.0f && g.z == 0.0f && g.w == 0.0f) return;
        float4 p = reinterpret_cast<float4*>(params)[i], m = reinterpret_cast<float4*>(exp_avg)[i],
               v = reinterpret_cast<float4*>(exp_avg_sq)[i];
        adamw_update(a, skip_zero, g.x, p.x, m.x, v.x);
        adamw_update(a, skip_zero, g.y, p.y, m.y, v.y);
        adamw_update(a, skip_zero, g.z, p.z, m.z, v.z);
        adamw_update(a, skip_zero, g.w, p.w, m.w, v.w);
        reinterpret_cast<float4*>(params)[i] = p;
        reinterpret_cast<float4*>(exp_avg)[i] = m;
        reinterpret_cast<float4*>(exp_avg_sq)[i] = v;
    } else {
        if (i >= n) return;
        float p = params[i], m = exp_avg[i], v = exp_avg_sq[i];
        const float g = grads[i];
        if (skip_zero && g == 0.0f) return;
        adamw_update(a, skip_zero, g, p, m, v);
        params[i] = p;
        exp_avg[i] = m;
        exp_avg_sq[i] = v;
    }
}

// The same update, or only the clearing of the gradient, restricted to the slot ranges a caller's map of
// touched ranges names (the sparse entry points): one workgroup per (slot range, level) looks at the
// range's flags (one per pair of features) and leaves at once when nothing was added there, so the
// cost follows what the batch touched and not the size of the table.  Within a touched range an entry
// with a gradient of exactly 0 is left alone, as with skip_zero.  `clear` zeroes the gradients the
// workgroup has used and the range's flags, which is what the next accumulation expects.
template <bool kUpdate, typename Vec>
__global__ void __launch_bounds__(kBlock)
touched_ranges_kernel(float* __restrict__ params, float* __restrict__ grads, float* __restrict__ exp_avg,
                      float* __restrict__ exp_avg_sq, uint32_t capacity, uint32_t nr_feat, uint32_t n_ranges,
                      uint32_t range_shift, uint32_t* __restrict__ touched, AdamWStep a, int clear) {
    constexpr uint32_t kPer = sizeof(Vec) / sizeof(float);
    const uint32_t range = blockIdx.x, level = blockIdx.y, pairs = nr_feat / 2;
    uint32_t any = 0u;
    for (uint32_t p = 0; p < pairs; ++p) any |= touched[(static_cast<size_t>(level) * pairs + p) * n_ranges + range];
    if (any == 0u) return;
    const uint32_t slot0 = range << range_shift;
    const uint32_t slots = capacity - slot0 < (1u << range_shift) ? capacity - slot0 : (1u << range_shift);
    const size_t base = (static_cast<size_t>(level) * capacity + slot0) * nr_feat;  // a multiple of kPer floats (the host checks)
    const uint32_t n_vec = slots * nr_feat / kPer;
    Vec* const g_at = reinterpret_cast<Vec*>(grads + base);
    for (uint32_t i = threadIdx.x; i < n_vec; i += kBlock) {
        const Vec gv = g_at[i];
        float g[kPer];
        __builtin_memcpy(g, &gv, sizeof(gv));
        bool nonzero = false;
#pragma unroll
        for (uint32_t k = 0; k < kPer; ++k) nonzero = nonzero || g[k] != 0.0f;
        if (!nonzero) continue;
        if constexpr (kUpdate) {
            Vec pv = reinterpret_cast<Vec*>(params + base)[i], mv = reinterpret_cast<Vec*>(exp_avg + base)[i],
                vv = reinterpret_cast<Vec*>(exp_avg_sq + base)[i];
            float p[kPer], m[kPer], v[kPer];
            __builtin_memcpy(p, &pv, sizeof(pv));
            __builtin_memcpy(m, &mv, sizeof(mv));
            __builtin_memcpy(v, &vv, sizeof(vv));
#pragma unroll
            for (uint32_t k = 0; k < kPer; ++k) adamw_update(a, true, g[k], p[k], m[k], v[k]);
            __builtin_memcpy(&pv, p, sizeof(pv));
            __builtin_memcpy(&mv, m, sizeof(mv));
            __builtin_memcpy(&vv, v, sizeof(vv));
            reinterpret_cast<Vec*>(params + base)[i] = pv;
            reinterpret_cast<Vec*>(exp_avg + base)[i] = mv;
            reinterpret_cast<Vec*>(exp_avg_sq + base)[i] = vv;
        }
        if (clear) {
            Vec zero;
            __builtin_memset(&zero, 0, sizeof(zero));
            g_at[i] = zero;
        }
    }
    if (clear) {
        __syncthreads();  // every thread has read the flags
        if (threadIdx.x < pairs) touched[(static_cast<size_t>(level) * pairs + threadIdx.x) * n_ranges + range] = 0u;
    }
}

// ------------------------------------------------------------------------------------------
// introspection

// kViaLds selects which of the two equivalent device routines produce the slots and weights: the
// compare-and-select chains (vertex_hashes / barycentric: table backward, position backward) or
// the thread-private LDS column (sort_by_rank_lds: forward, grad-of-grad).
template <int D, bool kViaLds>
__global__ void __launch_bounds__(kBlock)
simplex_debug_kernel(int n_points, uint32_t capacity, uint32_t cap_mask, const float* __restrict__ positions,
                     const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                     int* __restrict__ rem0, int* __restrict__ rank, int* __restrict__ slot,
                     float* __restrict__ bary) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    const int level = blockIdx.y;
    const Located<D> s = locate<D>(load_point<D>(positions, n), random_shift + level * D, scale_factor + level * D);
    uvec<D + 1> h;
    fvec<D + 1> w;
    if constexpr (kViaLds) {
        __shared__ uint2 columns[(D + 1) * kBlock];
        fvec<D + 1> sorted;
        sort_by_rank_lds<D>(columns + threadIdx.x, kBlock, s.rank, s.delta, s.hash0, sorted, h);
        w = barycentric_of_sorted<D>(sorted);
    } else {
        h = vertex_hashes<D>(s.rank, s.hash0);
        w = barycentric<D>(s.rank, s.delta);
    }
    const size_t o = (static_cast<size_t>(level) * n_points + n) * (D + 1);
    static_for<D + 1>(PENC_BODY(i) {
        PENC_INDEX(i);
        if (rem0) rem0[o + i] = s.rem0[i];
        if (rank) rank[o + i] = s.rank[i];
        if (slot) slot[o + i] = static_cast<int>(to_slot(h[i], capacity, cap_mask));
        if (bary) bary[o + i] = w[i];
    });
}

// dst[c][r] = src[r][c] for a tall matrix (rows = points, cols = 2 * levels): what turns the
// row-major upstream gradient (N, 2L) an MLP delivers into the level-major (L, 2, N) layout the
// kernels read (the reference does this with a strided `.contiguous()` copy,
// src/pytorch_modules/funcs.py:47).  Each workgroup moves kTransposeRows rows through LDS: the
// read is one contiguous chunk, every write a run of 64 consecutive floats.
constexpr int kTransposeRows = 64;  // rows per workgroup: one wavefront-wide run per written column

__global__ void __launch_bounds__(kBlock)
transpose_kernel(const float* __restrict__ src, int64_t src_row_stride, float* __restrict__ dst, int64_t rows, int cols) {
    extern __shared__ float tile[];  // kTransposeRows x (cols | 1)
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kTransposeRows;
    const int n_rows = rows - row0 < kTransposeRows ? static_cast<int>(rows - row0) : kTransposeRows;
    const int stride = cols | 1;  // odd: a column read walks all banks
    const float* chunk = src + row0 * src_row_stride;
    const int n_values = n_rows * cols;
    int r = threadIdx.x / cols, c = threadIdx.x % cols;
    const int dr = kBlock / cols, dc = kBlock % cols;
    for (int i = threadIdx.x; i < n_values; i += kBlock) {
        tile[r * stride + c] = chunk[r * src_row_stride + c];
        r += dr;
        c += dc;
        if (c >= cols) {
            c -= cols;
            ++r;
        }
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < n_rows)
        for (int col = wave; col < cols; col += kBlock / 64) dst[static_cast<int64_t>(col) * rows + row0 + lane] = tile[lane * stride + col];
}

// The other direction: dst[r][c] = src[c][r], from the [level][feature][n] layout the forward writes to rows
// dst[n][F * level + feature] of `dst_row_stride` floats (what a layer that wants contiguous rows reads; the
// reference's permute + reshape, src/pytorch_modules/modules.py:87, leaves that copy to the consumer).  Every
// read is a run of 64 consecutive floats, the write one contiguous chunk when the rows are dense.
__global__ void __launch_bounds__(kBlock)
transpose_to_rows_kernel(const float* __restrict__ src, float* __restrict__ dst, int64_t dst_row_stride, int64_t rows, int cols) {
    extern __shared__ float tile[];  // kTransposeRows x (cols | 1)
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kTransposeRows;
    const int n_rows = rows - row0 < kTransposeRows ? static_cast<int>(rows - row0) : kTransposeRows;
    const int stride = cols | 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < n_rows)
        for (int col = wave; col < cols; col += kBlock / 64)
            tile[lane * stride + col] = __builtin_nontemporal_load(src + static_cast<int64_t>(col) * rows + row0 + lane);
    __syncthreads();
    float* chunk = dst + row0 * dst_row_stride;
    const int n_values = n_rows * cols;
    int r = threadIdx.x / cols, c = threadIdx.x % cols;
    const int dr = kBlock / cols, dc = kBlock % cols;
    for (int i = threadIdx.x; i < n_values; i += kBlock) {
        chunk[r * dst_row_stride + c] = tile[r * stride + c];
        r += dr;
        c += dc;
        if (c >= cols) {
            c -= cols;
            ++r;
        }
    }
}

// Clears two arrays (the second may be empty): n2 and m2 count 8-byte units.
__global__ void __launch_bounds__(kBlock) fill_zero_kernel(float2* __restrict__ p, size_t n2, float2* __restrict__ q, size_t m2) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock, first = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    for (size_t i = first; i < n2; i += stride) p[i] = make_float2(0.0f, 0.0f);
    for (size_t i = first; i < m2; i += stride) q[i] = make_float2(0.0f, 0.0f);
}

// ------------------------------------------------------------------------------------------
// Scratch of penc_backward_static: device memory that is part of the loaded code object, so that
// callers who must not allocate (HIP graph capture, serving loops) still get the binned scatter.
// Every GPU the library runs on holds its own copy until the process ends.  In host code the
// array's name is only a handle for hipGetSymbolAddress: its device address is looked up once per
// device (static_scratch_of) and that pointer is what the launchers pass on.
static __device__ __align__(256) unsigned char scratch[PENC_STATIC_SCRATCH_BYTES];

// ------------------------------------------------------------------------------------------
// host side

inline int check_launch() { return hipGetLastError() == hipSuccess ? PENC_OK : PENC_ERR_LAUNCH; }

inline uint32_t mask_of(int capacity) {
    const uint32_t c = static_cast<uint32_t>(capacity);
    return (c & (c - 1)) == 0 ? c - 1 : 0u;
}

inline int check_geometry(int pos_dim, int nr_feat, int64_t n, int levels, int capacity, int extra) {
    if (pos_dim < 2 || pos_dim > 8) return PENC_ERR_UNSUPPORTED_POS_DIM;
    if (nr_feat != 2 && nr_feat != 4 && nr_feat != 8) return PENC_ERR_UNSUPPORTED_NR_FEAT;
    if (n <= 0 || levels <= 0 || capacity <= 0) return PENC_ERR_BAD_SIZE;
    const int64_t lim = (int64_t{1} << 31) - 1;
    if (n > lim / (nr_feat * (int64_t{levels} + extra)) || n > lim / pos_dim) return PENC_ERR_BAD_SIZE;
    if (int64_t{capacity} > lim / (nr_feat * int64_t{levels})) return PENC_ERR_BAD_SIZE;
    if (levels + extra > 65535) return PENC_ERR_BAD_SIZE;
    return PENC_OK;
}

inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
// The table as the gathering kernels see it: fp32 (format 0), or 16 bits per value (the *_half entry
// points: PENC_TABLE_FP16 or PENC_TABLE_BF16).
struct TableRef {
    const void* values;
    int format;
};
// a slot is gathered with one load (two of 16 bytes for eight floats): 4 to 16 bytes
inline bool table_aligned(const TableRef& t, int nr_feat) {
    const unsigned slot_bytes = static_cast<unsigned>(nr_feat) * (t.format != 0 ? 2u : 4u);
    return (reinterpret_cast<uintptr_t>(t.values) & ((slot_bytes < 16u ? slot_bytes : 16u) - 1u)) == 0;
}

// Clears the table gradient, and the bins' `direct` flags when there are bins (`flags` of
// `flag_bytes`, a multiple of 8), with a fill kernel (float2 granularity: the gradient is only
// guaranteed 8-byte alignment).  A kernel rather than hipMemsetAsync so that callers may capture
// the call in a HIP graph.
inline int clear_table_grad(float* g, int pair_levels, int capacity, void* flags, size_t flag_bytes, hipStream_t st) {
    const size_t n2 = static_cast<size_t>(pair_levels) * capacity;
    const size_t want = (n2 + kBlock * 8 - 1) / (kBlock * 8);
    const unsigned blocks = static_cast<unsigned>(want < 8192 ? want : 8192);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(kBlock), 0, st, reinterpret_cast<float2*>(g), n2,
                       static_cast<float2*>(flags), flags != nullptr ? flag_bytes / sizeof(float2) : size_t{0});
    return check_launch();
}

// How a workspace is cut into slot-range bins (see penc_scatter.hpp).  The levels are processed in
// passes of `levels_per_pass`; every pass reuses the same bins, so a smaller workspace means more,
// shorter passes (whose records are more likely still in cache when they are read back), not less
// binning.
struct BinPlan {
    bool enabled = false;
    int levels_per_pass = 0;
    BinTarget target{};       // of the first pass; target.direct covers all levels, a pass starts at its first level's flags
    size_t direct_bytes = 0;  // size of target.direct (to be cleared with the gradient)
};

// Bytes of the `direct` flags of all levels (one 4-byte flag per level and bin), padded to the workspace's alignment.
inline size_t direct_flag_bytes(int levels, uint32_t n_bins) {
    return (static_cast<size_t>(levels) * n_bins * sizeof(uint32_t) + 255u) & ~size_t{255};
}

// log2 of the slots per bin: kBinSlotsLog2 (what a reducer workgroup's LDS holds) up to kMaxBins bins, wider
// bins (summed one LDS-full after the other) for larger tables, up to kMaxBinSlotsLog2.
inline uint32_t bin_shift_for_capacity(int capacity) {
    uint32_t shift = kBinSlotsLog2;
    while (shift < static_cast<uint32_t>(kMaxBinSlotsLog2) &&
           ((static_cast<int64_t>(capacity) + (int64_t{1} << shift) - 1) >> shift) > kMaxBins)
        ++shift;
    return shift;
}

// Bins per level; more than kMaxBins means the table is too large for binning.
inline uint32_t bins_for_capacity(int capacity) {
    const uint32_t shift = bin_shift_for_capacity(capacity);
    return static_cast<uint32_t>((static_cast<int64_t>(capacity) + (int64_t{1} << shift) - 1) >> shift);
}

constexpr int64_t kMinSlotsPerContribution = 8;
constexpr int64_t kLargeGroupsMinWorkgroups = 3000;  // about four per workgroup slot of the chip (256 CUs x 3)

inline unsigned scatter_groups(int64_t n, int tiles_per_group) {
    const int64_t group_points = static_cast<int64_t>(tiles_per_group) * kScatterBlock;
    return static_cast<unsigned>((n + group_points - 1) / group_points);
}

// Tiles per scattering workgroup of the table backward.  Larger groups mean longer record segments
// (less slack, longer bursts for the reducer) and fewer cache flushes; they are taken when the
// launch still has several workgroups for every slot of the chip (measured: 3-13% faster then,
// slower otherwise).  The same rule serves the scattering half of the double backward.
// Small batches take smaller groups, down to two tiles, until the launch has a workgroup for every slot of
// the chip (measured at 24 levels, D = 3: 2^16 points 0.074 -> 0.064 ms with four tiles, 2^15 points
// 0.065 -> 0.055 ms and 2^14 points 0.062 -> 0.048 ms with two; 2^17 points are best with eight).
constexpr int64_t kMinWorkgroups = 768;  // three per compute unit
inline int table_backward_tiles(int64_t n, int levels) {
    if (static_cast<int64_t>(scatter_groups(n, kScatterTilesLarge)) * levels >= kLargeGroupsMinWorkgroups) return kScatterTilesLarge;
    int tiles = kScatterTiles;
    while (tiles > 2 && static_cast<int64_t>(scatter_groups(n, tiles)) * levels < kMinWorkgroups) tiles /= 2;
    return tiles;
}

// Split records (10 bytes in two arrays) where a tile's records leave in long runs (the
// workgroup-wide sort), whole ones (12 bytes) elsewhere (see BinRecord).
inline size_t record_bytes(int pos_dim, uint32_t n_bins) {
    return pos_dim <= kWorkgroupSortMaxDim && n_bins <= static_cast<uint32_t>(kStageBins) ? kSplitRecordBytes : sizeof(BinRecord);
}

// Records one scattering workgroup may leave in one bin: its share of the
// group's contributions (D+1 per point) plus the flushed cache lines, with three standard deviations
// of a uniform hash on top.  A segment that still overflows spills to direct atomics.
inline uint32_t wanted_segment_capacity(int pos_dim, uint32_t n_bins, int tiles_per_group) {
    const double mean = (static_cast<double>(tiles_per_group) * kScatterBlock * (pos_dim + 1) + kCacheLines) / n_bins;
    const uint32_t cap = static_cast<uint32_t>(mean + 3.0 * __builtin_sqrt(mean) + 8.0);
    // split records: a multiple of four per segment keeps every segment's values 16-byte aligned
    return record_bytes(pos_dim, n_bins) == kSplitRecordBytes ? (cap + 3u) & ~3u : cap;
}

inline size_t bin_bytes_per_level(int pos_dim, uint32_t n_bins, uint32_t n_groups, uint32_t segment_capacity) {
    const size_t segments = static_cast<size_t>(n_bins) * n_groups;
    return segments * (sizeof(uint32_t) + static_cast<size_t>(segment_capacity) * record_bytes(pos_dim, n_bins));
}

inline BinPlan plan_bins(int pos_dim, int64_t n, int levels, int capacity, int tiles_per_group, void* workspace,
                         size_t bytes) {
    BinPlan p;
    const uint32_t n_bins = bins_for_capacity(capacity);
    const uint32_t n_groups = scatter_groups(n, tiles_per_group);
    if (workspace == nullptr || n_bins > static_cast<uint32_t>(kMaxBins)) return p;
    // few contributions per slot: the reducer's fixed cost per bin (clearing and flushing 128 KiB of
    // LDS) exceeds what direct atomics cost (measured crossover: one contribution per eight slots)
    if (n * (pos_dim + 1) * kMinSlotsPerContribution <= capacity) return p;
    const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255u) & ~uintptr_t{255};
    const size_t lost = base - reinterpret_cast<uintptr_t>(workspace);
    const size_t flag_bytes = direct_flag_bytes(levels, n_bins);
    if (bytes < lost + flag_bytes + 4096) return p;
    bytes -= lost + flag_bytes + 256;
    const size_t segments = static_cast<size_t>(n_bins) * n_groups;
    const bool split = record_bytes(pos_dim, n_bins) == kSplitRecordBytes;
    uint32_t cap = wanted_segment_capacity(pos_dim, n_bins, tiles_per_group);
    if (bytes < bin_bytes_per_level(pos_dim, n_bins, n_groups, cap)) {  // not even one level at the wanted size: shrink the segments
        if (bytes < segments * (sizeof(uint32_t) + 16 * record_bytes(pos_dim, n_bins))) return p;
        cap = static_cast<uint32_t>((bytes / segments - sizeof(uint32_t)) / record_bytes(pos_dim, n_bins));
        if (split) cap &= ~3u;
    }
    // the scattering kernel addresses a level's records with 32-bit byte offsets
    const uint64_t max_records_per_level = 0xFFFFFFFFull / (split ? sizeof(RecordValues) : sizeof(BinRecord));
    if (segments * cap > max_records_per_level) {
        cap = static_cast<uint32_t>(max_records_per_level / segments);
        if (split) cap &= ~3u;
        if (cap < 16) return p;
    }
    const size_t fit = bytes / bin_bytes_per_level(pos_dim, n_bins, n_groups, cap);
    p.levels_per_pass = static_cast<int>(fit < static_cast<size_t>(levels) ? fit : static_cast<size_t>(levels));
    // wide bins are served by bin_reduce_levels_kernel only
    if (bin_shift_for_capacity(capacity) != static_cast<uint32_t>(kBinSlotsLog2) &&
        (cap > kLevelsMaxSegment || n_groups > static_cast<uint32_t>(kReduceBlock)))
        return p;
    p.target.n_bins = n_bins;
    p.target.n_groups = n_groups;
    p.target.segment_capacity = cap;
    p.target.bin_shift = bin_shift_for_capacity(capacity);
    p.target.direct = reinterpret_cast<uint32_t*>(base);
    p.direct_bytes = flag_bytes;
    const uintptr_t counts_at = base + flag_bytes;
    p.target.counts = reinterpret_cast<uint32_t*>(counts_at);
    const size_t counts_bytes = (static_cast<size_t>(p.levels_per_pass) * segments * sizeof(uint32_t) + 255u) & ~size_t{255};
    const size_t records_per_pass = static_cast<size_t>(p.levels_per_pass) * segments * cap;
    p.target.records = reinterpret_cast<void*>(counts_at + counts_bytes);
    p.target.slots = split ? reinterpret_cast<uint16_t*>(counts_at + counts_bytes + records_per_pass * sizeof(RecordValues)) : nullptr;
    p.enabled = true;
    return p;
}

// Running consecutive passes on two streams (scatter pass p+1 while pass p is reduced) was tried and
// measured 10-15% slower than one pass over all levels on one stream; hence a single stream.
constexpr unsigned kReduceWorkgroupsWanted = 512;  // two per compute unit
constexpr unsigned kMaxReduceSplits = 16;

inline int reduce_bins(const BinPlan& p, const float* window, int first_level, int n_levels_in_pass, int capacity,
                       uint32_t feat_pairs, float* table_grad, hipStream_t st) {
    // enough workgroups for every compute unit, by letting several share a bin when bins*levels is small
    const unsigned pairs = p.target.n_bins * static_cast<unsigned>(n_levels_in_pass);
    unsigned splits = pairs >= kReduceWorkgroupsWanted ? 1u : (kReduceWorkgroupsWanted + pairs - 1) / pairs;
    if (splits > p.target.n_groups) splits = p.target.n_groups;
    if (splits > kMaxReduceSplits) splits = kMaxReduceSplits;
    // many bins with a few thousand records each: workgroups that keep their bin and walk several levels
    // (bins wider than kBinSlots are planned only where this kernel can serve them)
    const bool wide = p.target.bin_shift != static_cast<uint32_t>(kBinSlotsLog2);
    if (wide || (p.target.slots == nullptr && p.target.n_bins > static_cast<uint32_t>(kStageBins) && splits == 1 &&
                 p.target.segment_capacity <= kLevelsMaxSegment && p.target.n_groups <= static_cast<uint32_t>(kReduceBlock))) {
        const unsigned levels = static_cast<unsigned>(n_levels_in_pass);
        unsigned per_bin = (levels + kLevelsMaxPerWorkgroup - 1) / kLevelsMaxPerWorkgroup;
        const unsigned to_fill = (kReduceWorkgroupsWanted + p.target.n_bins - 1) / p.target.n_bins;  // two workgroups per compute unit, one after the other
        if (per_bin < to_fill) per_bin = to_fill;
        if (per_bin > levels) per_bin = levels;
        hipLaunchKernelGGL(bin_reduce_levels_kernel, dim3(p.target.n_bins, per_bin), dim3(kReduceBlock), 0, st, p.target, window,
                           static_cast<uint32_t>(capacity), feat_pairs, table_grad, first_level, static_cast<uint32_t>(levels));
        return check_launch();
    }
    const dim3 grid(p.target.n_bins, n_levels_in_pass, splits);
    if (p.target.slots != nullptr)
        hipLaunchKernelGGL(bin_reduce_kernel<true>, grid, dim3(kReduceBlock), 0, st, p.target, window,
                           static_cast<uint32_t>(capacity), feat_pairs, table_grad, first_level);
    else
        hipLaunchKernelGGL(bin_reduce_kernel<false>, grid, dim3(kReduceBlock), 0, st, p.target, window,
                           static_cast<uint32_t>(capacity), feat_pairs, table_grad, first_level);
    return check_launch();
}

#define PENC_DISPATCH_D(D_, ...)                                  \
    switch (D_) {                                                  \
        case 2: { constexpr int DD = 2; __VA_ARGS__; } break;      \
        case 3: { constexpr int DD = 3; __VA_ARGS__; } break;      \
        case 4: { constexpr int DD = 4; __VA_ARGS__; } break;      \
        case 5: { constexpr int DD = 5; __VA_ARGS__; } break;      \
        case 6: { constexpr int DD = 6; __VA_ARGS__; } break;      \
        case 7: { constexpr int DD = 7; __VA_ARGS__; } break;      \
        case 8: { constexpr int DD = 8; __VA_ARGS__; } break;      \
        default: return PENC_ERR_UNSUPPORTED_POS_DIM;              \
    }

// The same with the number of features per level (2, 4 or 8) as the constant FF.
#define PENC_DISPATCH_DF(D_, F_, ...)                                   \
    if ((F_) == 8) {                                                    \
        constexpr int FF = 8;                                           \
        PENC_DISPATCH_D(D_, __VA_ARGS__)                                \
    } else if ((F_) == 4) {                                             \
        constexpr int FF = 4;                                           \
        PENC_DISPATCH_D(D_, __VA_ARGS__)                                \
    } else {                                                            \
        constexpr int FF = 2;                                           \
        PENC_DISPATCH_D(D_, __VA_ARGS__)                                \
    }

// The same with the table's element type (float, __half or bfloat16_bits) as TT.
#define PENC_DISPATCH_DFT(D_, F_, FORMAT_, ...)                         \
    if ((FORMAT_) == PENC_TABLE_BF16) {                                 \
        using TT = bfloat16_bits;                                       \
        PENC_DISPATCH_DF(D_, F_, __VA_ARGS__)                           \
    } else if ((FORMAT_) == PENC_TABLE_FP16) {                          \
        using TT = __half;                                              \
        PENC_DISPATCH_DF(D_, F_, __VA_ARGS__)                           \
    } else {                                                            \
        using TT = float;                                               \
        PENC_DISPATCH_DF(D_, F_, __VA_ARGS__)                           \
    }

inline unsigned tiles(int64_t n) { return static_cast<unsigned>((n + kBlock - 1) / kBlock); }

// Levels a thread of the forward and of the gathering half of the double backward takes: two up to
// pos_dim 4 (measured on the forward at 2^20 points, 24 levels: 0.310 -> 0.302 ms at pos_dim 3, 0.275 -> 0.259 ms with a
// 2^22-slot table, 0.396 -> 0.392 ms at pos_dim 4; at pos_dim 8 0.283 -> 0.298 ms).
inline int gather_levels_per_thread(int pos_dim) { return pos_dim <= 4 ? 2 : 1; }

// Device address of this GPU's copy of `scratch`, looked up on the first call with that GPU
// current and kept for the life of the process.  Returns nullptr when the lookup fails.
constexpr int kMaxDevices = 64;
inline void* static_scratch_of_current_device() {
    static std::mutex lock;
    static void* address[kMaxDevices] = {};
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> guard(lock);
    if (address[device] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) {
            (void)hipGetLastError();  // the failure is reported by the caller's status code, not by a later launch check
            return nullptr;
        }
        address[device] = p;
    }
    return address[device];
}

// Accelerator dies of the current GPU (each with an L2 of its own; workgroup i of a launch runs on
// die i % dies), asked of the runtime once per device.  kDefaultDies when the runtime does not say.
inline uint32_t dies_of_current_device() {
    static std::mutex lock;
    static uint32_t dies[kMaxDevices] = {};
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return kDefaultDies;
    std::lock_guard<std::mutex> guard(lock);
    if (dies[device] == 0u) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeNumberOfXccs, device) != hipSuccess) {
            (void)hipGetLastError();
            n = 0;
        }
        dies[device] = n >= 1 && n <= 64 ? static_cast<uint32_t>(n) : kDefaultDies;
    }
    return dies[device];
}

}  // namespace penc

using namespace penc;

// The table gradient of penc_backward / penc_backward_table_rowmajor: clear, scatter, reduce the
// bins, in as many passes over the levels as the workspace asks for.  grad_row_stride == 0 means
// the [level][feature][n] layout, otherwise the gradient is rows of that many floats.  With
// double_pos_grad the same for the table-gradient half of the double backward.  grad_level_major (rows
// only, may be NULL) receives the upstream gradient in [level][feature][n] order as a by-product.
// With `touched` (the sparse entry points) nothing is cleared: the sums are added to a gradient the caller
// keeps across calls, and `touched` [pair level][slot range] is that caller's record of the slot ranges
// that hold anything; it takes the place of the workspace's flags of direct adds.
static int table_backward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity, const float* positions,
                          const float* scale_factor, const float* random_shift, const float* anneal_window,
                          const float* grad, int64_t grad_row_stride, const float* double_pos_grad,
                          float* lattice_values_grad, float* grad_level_major, void* workspace, size_t workspace_bytes,
                          hipStream_t st, uint32_t* touched = nullptr) {
    const int n = static_cast<int>(nr_positions);
    const uint32_t cap = static_cast<uint32_t>(capacity), mask = mask_of(capacity);
    // every pair of features is scattered like a level of its own (see backward_table_kernel)
    const uint32_t feat_pairs = static_cast<uint32_t>(nr_feat / 2);
    const int pair_levels = nr_levels * static_cast<int>(feat_pairs);
    int tiles_per_group = table_backward_tiles(nr_positions, pair_levels);
    BinPlan plan = plan_bins(pos_dim, nr_positions, pair_levels, capacity, tiles_per_group, workspace, workspace_bytes);
    if (!plan.enabled && tiles_per_group > kScatterTiles) {  // wide bins need short segments: smaller groups of points
        tiles_per_group = kScatterTiles;
        plan = plan_bins(pos_dim, nr_positions, pair_levels, capacity, tiles_per_group, workspace, workspace_bytes);
    }
    if (touched != nullptr) {
        plan.target.direct = touched;
        plan.target.n_bins = bins_for_capacity(capacity);
        plan.target.bin_shift = bin_shift_for_capacity(capacity);
    } else if (int rc = clear_table_grad(lattice_values_grad, pair_levels, capacity, plan.enabled ? plan.target.direct : nullptr,
                                         plan.direct_bytes, st)) {
        return rc;
    }
    uint32_t* const direct_flags = plan.target.direct;
    const int per_pass = plan.enabled ? plan.levels_per_pass : pair_levels;
    const uint32_t dies = dies_of_current_device();
    for (int first = 0; first < pair_levels; first += per_pass) {
        const int count = pair_levels - first < per_pass ? pair_levels - first : per_pass;
        const unsigned padded_groups = (scatter_groups(nr_positions, tiles_per_group) + dies - 1) / dies * dies;
        const dim3 grid(padded_groups * static_cast<unsigned>(count));
        if (direct_flags != nullptr) plan.target.direct = direct_flags + static_cast<size_t>(first) * plan.target.n_bins;
#define PENC_LAUNCH_TABLE_(ROW_MAJOR, SECOND_ORDER, WIDE)                                                                  \
    PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((backward_table_kernel<DD, ROW_MAJOR, SECOND_ORDER, WIDE>), grid,            \
                                                dim3(kScatterBlock), 0, st, n, first, static_cast<uint32_t>(count),          \
                                                feat_pairs, dies, tiles_per_group, cap, mask, positions, scale_factor,       \
                                                random_shift, anneal_window, grad, grad_row_stride, double_pos_grad,         \
                                                lattice_values_grad, grad_level_major, plan.target))
#define PENC_LAUNCH_TABLE(ROW_MAJOR, SECOND_ORDER)       \
    if (wide_bins) {                                     \
        PENC_LAUNCH_TABLE_(ROW_MAJOR, SECOND_ORDER, true);  \
    } else {                                             \
        PENC_LAUNCH_TABLE_(ROW_MAJOR, SECOND_ORDER, false); \
    }
        const bool wide_bins = direct_flags != nullptr && plan.target.bin_shift != static_cast<uint32_t>(kBinSlotsLog2);
        if (double_pos_grad != nullptr && grad_row_stride != 0) {
            PENC_LAUNCH_TABLE(true, true);
        } else if (double_pos_grad != nullptr) {
            PENC_LAUNCH_TABLE(false, true);
        } else if (grad_row_stride != 0) {
            PENC_LAUNCH_TABLE(true, false);
        } else {
            PENC_LAUNCH_TABLE(false, false);
        }
#undef PENC_LAUNCH_TABLE
#undef PENC_LAUNCH_TABLE_
        if (int rc = check_launch()) return rc;
        if (plan.enabled)
            if (int rc = reduce_bins(plan, anneal_window, first, count, capacity, feat_pairs, lattice_values_grad, st)) return rc;
    }
    return PENC_OK;
}

// The position gradient of penc_backward / penc_backward_rowmajor from a level-major upstream gradient:
// levels in groups of pos_levels_per_group() when the workspace can hold the partial sums, else one
// thread per point walks all levels.
static int positions_backward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity, const float* positions,
                              const TableRef& table, const float* scale_factor, const float* random_shift,
                              const float* anneal_window, const float* grad_level_major, float* positions_grad,
                              void* workspace, size_t workspace_bytes, hipStream_t st) {
    const int n = static_cast<int>(nr_positions);
    const uint32_t cap = static_cast<uint32_t>(capacity), mask = mask_of(capacity);
    const size_t n_values = static_cast<size_t>(nr_positions) * pos_dim;
    int per_group = nr_levels, groups = 1;
    float* partial = positions_grad;
    const uintptr_t ws = (reinterpret_cast<uintptr_t>(workspace) + 255u) & ~uintptr_t{255};
    const int want_groups = (nr_levels + pos_levels_per_group(pos_dim) - 1) / pos_levels_per_group(pos_dim);
    if (workspace != nullptr && want_groups > 1 &&
        workspace_bytes >= (ws - reinterpret_cast<uintptr_t>(workspace)) + want_groups * n_values * sizeof(float)) {
        per_group = pos_levels_per_group(pos_dim);
        groups = want_groups;
        partial = reinterpret_cast<float*>(ws);
    }
    PENC_DISPATCH_DFT(pos_dim, nr_feat, table.format,
                      hipLaunchKernelGGL((backward_pos_kernel<DD, FF, TT>), dim3(tiles(nr_positions), groups), dim3(kBlock), 0,
                                         st, n, nr_levels, per_group, cap, mask, positions,
                                         static_cast<const TT*>(table.values), scale_factor, random_shift, anneal_window,
                                         grad_level_major, partial));
    if (int rc = check_launch()) return rc;
    if (groups > 1) {
        const size_t want = (n_values + kBlock * 4 - 1) / (kBlock * 4);
        hipLaunchKernelGGL(reduce_level_groups_kernel, dim3(static_cast<unsigned>(want < 8192 ? want : 8192)), dim3(kBlock),
                           0, st, partial, groups, n_values, positions_grad);
        if (int rc = check_launch()) return rc;
    }
    return PENC_OK;
}

static int transpose_rows(const float* src, int64_t src_row_stride, float* dst, int64_t rows, int cols, hipStream_t st) {
    const size_t lds = static_cast<size_t>(kTransposeRows) * (cols | 1) * sizeof(float);
    if (cols <= 0 || cols > 255 || lds > 64 * 1024) return PENC_ERR_BAD_SIZE;
    const unsigned blocks = static_cast<unsigned>((rows + kTransposeRows - 1) / kTransposeRows);
    hipLaunchKernelGGL(transpose_kernel, dim3(blocks), dim3(kBlock), lds, st, src, src_row_stride, dst, rows, cols);
    return check_launch();
}

static int transpose_to_rows(const float* src, float* dst, int64_t dst_row_stride, int64_t rows, int cols, hipStream_t st) {
    const size_t lds = static_cast<size_t>(kTransposeRows) * (cols | 1) * sizeof(float);
    if (cols <= 0 || cols > 255 || lds > 64 * 1024) return PENC_ERR_BAD_SIZE;
    const unsigned blocks = static_cast<unsigned>((rows + kTransposeRows - 1) / kTransposeRows);
    hipLaunchKernelGGL(transpose_to_rows_kernel, dim3(blocks), dim3(kBlock), lds, st, src, dst, dst_row_stride, rows, cols);
    return check_launch();
}

// penc_backward and penc_backward_static: argument checks, then the table gradient (clear, scatter,
// reduce) and the position gradient on the same stream.
static int backward_impl(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                         const float* positions, const TableRef& table, const float* scale_factor,
                         const float* random_shift, const float* anneal_window,
                         const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                         void* workspace, size_t workspace_bytes, void* stream, uint32_t* touched = nullptr) {
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, 0)) return rc;
    if (!positions || !scale_factor || !random_shift || !anneal_window || !grad_sliced_values)
        return PENC_ERR_NULL_POINTER;
    if (!lattice_values_grad && !positions_grad) return PENC_ERR_NULL_POINTER;
    if (positions_grad && !table.values) return PENC_ERR_NULL_POINTER;
    if ((table.values && !table_aligned(table, nr_feat)) || !aligned8(lattice_values_grad)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (lattice_values_grad)
        if (int rc = table_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, scale_factor, random_shift,
                                    anneal_window, grad_sliced_values, 0, nullptr, lattice_values_grad, nullptr, workspace,
                                    workspace_bytes, st, touched))
            return rc;
    if (positions_grad)
        return positions_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor,
                                  random_shift, anneal_window, grad_sliced_values, positions_grad, workspace, workspace_bytes, st);
    return PENC_OK;
}

static int forward_impl(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                        const float* positions, const TableRef& table, const float* scale_factor,
                        const float* random_shift, const float* anneal_window, float* sliced_values,
                        int concat_points, float points_scaling, void* stream) {
    const int extra = penc_extra_levels(pos_dim, nr_feat, concat_points);
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, extra)) return rc;
    if (!positions || !table.values || !scale_factor || !random_shift || !anneal_window || !sliced_values)
        return PENC_ERR_NULL_POINTER;
    if (!table_aligned(table, nr_feat)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int per_thread = gather_levels_per_thread(pos_dim);
    const dim3 grid(tiles(nr_positions), (nr_levels + extra + per_thread - 1) / per_thread);
    PENC_DISPATCH_DFT(pos_dim, nr_feat, table.format,
                      hipLaunchKernelGGL((forward_kernel<DD, FF, TT>), grid, dim3(kBlock), 0, st,
                                         static_cast<int>(nr_positions), nr_levels, nr_levels + extra, per_thread, static_cast<uint32_t>(capacity),
                                         mask_of(capacity), positions, static_cast<const TT*>(table.values), scale_factor,
                                         random_shift, anneal_window, sliced_values, points_scaling));
    return check_launch();
}

extern "C" {

const char* penc_status_string(int status) {
    switch (status) {
        case PENC_OK: return "ok";
        case PENC_ERR_NULL_POINTER: return "a required pointer is NULL";
        case PENC_ERR_BAD_SIZE: return "nr_positions, nr_levels and capacity must be positive and every array must stay below 2^31 elements";
        case PENC_ERR_UNSUPPORTED_POS_DIM: return "pos_dim must be 2,3,4,5,6,7 or 8";
        case PENC_ERR_UNSUPPORTED_NR_FEAT: return "nr_feat_per_level must be 2, 4 or 8";
        case PENC_ERR_MISALIGNED: return "lattice_values must be aligned to one slot (at most 16 bytes), lattice_values_grad and gradient rows to 8 bytes";
        case PENC_ERR_LAUNCH: return "the HIP runtime rejected a kernel launch";
        case PENC_ERR_WORKSPACE_TOO_SMALL: return "the workspace cannot hold the level-major array the call needs (penc_backward_rowmajor_workspace_bytes, penc_forward_rowmajor_workspace_bytes)";
        case PENC_ERR_UNSUPPORTED_TABLE_FORMAT: return "table_format must be PENC_TABLE_FP16 or PENC_TABLE_BF16";
        case PENC_ERR_SCRATCH_TOO_SMALL: return "the problem is too large for the library's static scratch (penc_static_scratch_bytes): use penc_backward with a workspace";
        default: return "unknown status";
    }
}

int penc_extra_levels(int pos_dim, int nr_feat, int concat_points) {
    if (!concat_points || nr_feat <= 0) return 0;
    return (pos_dim + nr_feat - 1) / nr_feat;
}

size_t penc_scatter_workspace_bytes(int pos_dim, int64_t nr_positions, int nr_levels, int capacity, int levels_per_pass) {
    if (pos_dim < 2 || pos_dim > 8 || nr_positions <= 0 || nr_levels <= 0 || capacity <= 0) return 0;
    const uint32_t n_bins = bins_for_capacity(capacity);
    if (n_bins > static_cast<uint32_t>(kMaxBins)) return 0;
    if (levels_per_pass <= 0) levels_per_pass = kDefaultLevelsPerPass;
    if (levels_per_pass > nr_levels) levels_per_pass = nr_levels;
    // the larger of what the two gradient calls plan for (they may group the points differently)
    size_t per_level = 0;
    for (const int tiles : {kScatterTiles, table_backward_tiles(nr_positions, nr_levels)}) {
        const size_t need = bin_bytes_per_level(pos_dim, n_bins, scatter_groups(nr_positions, tiles),
                                                wanted_segment_capacity(pos_dim, n_bins, tiles));
        per_level = need > per_level ? need : per_level;
    }
    return per_level * static_cast<size_t>(levels_per_pass) + direct_flag_bytes(nr_levels, n_bins) + 1024;
}

size_t penc_positions_workspace_bytes(int pos_dim, int64_t nr_positions, int nr_levels) {
    if (pos_dim < 2 || pos_dim > 8 || nr_positions <= 0 || nr_levels <= pos_levels_per_group(pos_dim)) return 0;
    const size_t groups = static_cast<size_t>((nr_levels + pos_levels_per_group(pos_dim) - 1) / pos_levels_per_group(pos_dim));
    return groups * static_cast<size_t>(nr_positions) * pos_dim * sizeof(float) + 256;
}

int penc_scale_factors(int pos_dim, int nr_levels, const float* sigmas, float* scale_factor_out) {
    if (!sigmas || !scale_factor_out) return PENC_ERR_NULL_POINTER;
    if (pos_dim < 1 || nr_levels < 1) return PENC_ERR_BAD_SIZE;
    for (int l = 0; l < nr_levels; ++l)
        for (int i = 0; i < pos_dim; ++i) {
            // the reference divides a float32 tensor element by a host scalar (Encoding.cuh:62-63), which ATen
            // evaluates as element * (1.0f / scalar): two roundings, up to one unit in the last place away
            // from a true division
            const float numerator = static_cast<float>(1.0 / __builtin_sqrt(static_cast<double>((i + 1) * (i + 2))));
            const float reciprocal = 1.0f / sigmas[l];
            scale_factor_out[l * pos_dim + i] = numerator * reciprocal;
        }
    return PENC_OK;
}

int penc_forward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                 const float* positions, const float* lattice_values, const float* scale_factor,
                 const float* random_shift, const float* anneal_window, float* sliced_values,
                 int concat_points, float points_scaling, void* stream) {
    return forward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                        scale_factor, random_shift, anneal_window, sliced_values, concat_points, points_scaling, stream);
}

size_t penc_forward_rowmajor_workspace_bytes(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int concat_points) {
    if (pos_dim < 2 || pos_dim > 8 || (nr_feat != 2 && nr_feat != 4 && nr_feat != 8) || nr_positions <= 0 || nr_levels <= 0) return 0;
    const size_t cols = static_cast<size_t>(nr_feat) * (nr_levels + penc_extra_levels(pos_dim, nr_feat, concat_points));
    return cols * static_cast<size_t>(nr_positions) * sizeof(float) + 256;
}

int penc_forward_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                          const float* positions, const float* lattice_values, const float* scale_factor,
                          const float* random_shift, const float* anneal_window, float* sliced_rows, int64_t row_stride,
                          int concat_points, float points_scaling, void* workspace, size_t workspace_bytes, void* stream) {
    const int extra = penc_extra_levels(pos_dim, nr_feat, concat_points);
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, extra)) return rc;
    if (!sliced_rows) return PENC_ERR_NULL_POINTER;
    const int cols = nr_feat * (nr_levels + extra);
    if (cols > 255 || row_stride < cols || row_stride * nr_positions >= (int64_t{1} << 31)) return PENC_ERR_BAD_SIZE;
    const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255u) & ~uintptr_t{255};
    const size_t need = static_cast<size_t>(cols) * static_cast<size_t>(nr_positions) * sizeof(float);
    if (workspace == nullptr || workspace_bytes < (base - reinterpret_cast<uintptr_t>(workspace)) + need) return PENC_ERR_WORKSPACE_TOO_SMALL;
    float* level_major = reinterpret_cast<float*>(base);
    if (int rc = forward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0}, scale_factor,
                              random_shift, anneal_window, level_major, concat_points, points_scaling, stream))
        return rc;
    return transpose_to_rows(level_major, sliced_rows, row_stride, nr_positions, cols, static_cast<hipStream_t>(stream));
}

int penc_forward_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                      const float* positions, const void* lattice_values_half, int table_format,
                      const float* scale_factor, const float* random_shift, const float* anneal_window,
                      float* sliced_values, int concat_points, float points_scaling, void* stream) {
    if (table_format != PENC_TABLE_FP16 && table_format != PENC_TABLE_BF16) return PENC_ERR_UNSUPPORTED_TABLE_FORMAT;
    return forward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values_half, table_format},
                        scale_factor, random_shift, anneal_window, sliced_values, concat_points, points_scaling, stream);
}

int penc_backward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                  const float* positions, const float* lattice_values, const float* scale_factor,
                  const float* random_shift, const float* anneal_window,
                  const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                  void* workspace, size_t workspace_bytes, void* stream) {
    return backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                         scale_factor, random_shift, anneal_window, grad_sliced_values, lattice_values_grad, positions_grad,
                         workspace, workspace_bytes, stream);
}

size_t penc_static_scratch_bytes(void) { return PENC_STATIC_SCRATCH_BYTES; }

int penc_backward_static(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                         const float* positions, const float* lattice_values, const float* scale_factor,
                         const float* random_shift, const float* anneal_window,
                         const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                         void* stream) {
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, 0)) return rc;
    // the scratch must hold the slot-range records of at least one level (more levels per pass as
    // they fit), a pair of features counting as a level; a problem the scatter does not bin (a capacity
    // beyond the bins' reach, too few contributions per slot) needs no scratch at all
    const int pair_levels = nr_levels * (nr_feat / 2);
    const bool binned = bins_for_capacity(capacity) <= static_cast<uint32_t>(kMaxBins) &&
                        nr_positions * (pos_dim + 1) * kMinSlotsPerContribution > capacity;
    if (lattice_values_grad != nullptr && binned &&
        penc_scatter_workspace_bytes(pos_dim, nr_positions, pair_levels, capacity, 1) > PENC_STATIC_SCRATCH_BYTES)
        return PENC_ERR_SCRATCH_TOO_SMALL;
    void* ws = static_scratch_of_current_device();
    if (ws == nullptr) return PENC_ERR_LAUNCH;
    return backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                         scale_factor, random_shift, anneal_window, grad_sliced_values, lattice_values_grad, positions_grad, ws,
                         PENC_STATIC_SCRATCH_BYTES, stream);
}

static int check_rows(const float* grad_rows, int64_t grad_row_stride, int64_t nr_positions, int nr_levels, int nr_feat) {
    if (!grad_rows) return PENC_ERR_NULL_POINTER;
    if (grad_row_stride < nr_feat * static_cast<int64_t>(nr_levels) || (grad_row_stride & 1) != 0 ||
        grad_row_stride * nr_positions >= (int64_t{1} << 31))
        return PENC_ERR_BAD_SIZE;
    if (!aligned8(grad_rows)) return PENC_ERR_MISALIGNED;
    return PENC_OK;
}

size_t penc_backward_rowmajor_workspace_bytes(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                              int want_lattice_values_grad, int want_positions_grad) {
    if (pos_dim < 2 || pos_dim > 8 || (nr_feat != 2 && nr_feat != 4 && nr_feat != 8) || nr_positions <= 0 || nr_levels <= 0 || capacity <= 0)
        return 0;
    size_t scratch = 0;
    if (want_lattice_values_grad)
        scratch = penc_scatter_workspace_bytes(pos_dim, nr_positions, nr_levels * (nr_feat / 2), capacity, 0);
    if (!want_positions_grad) return scratch;
    const size_t partial = penc_positions_workspace_bytes(pos_dim, nr_positions, nr_levels);
    const size_t copy = static_cast<size_t>(nr_levels) * nr_feat * static_cast<size_t>(nr_positions) * sizeof(float);
    return 512 + copy + (scratch > partial ? scratch : partial);
}

static int backward_rowmajor_impl(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                  const float* positions, const TableRef& table, const float* scale_factor,
                                  const float* random_shift, const float* anneal_window, const float* grad_rows,
                                  int64_t grad_row_stride, float* lattice_values_grad, float* positions_grad,
                                  void* workspace, size_t workspace_bytes, void* stream, uint32_t* touched = nullptr) {
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, 0)) return rc;
    if (!positions || !scale_factor || !random_shift || !anneal_window) return PENC_ERR_NULL_POINTER;
    if (!lattice_values_grad && !positions_grad) return PENC_ERR_NULL_POINTER;
    if (positions_grad && !table.values) return PENC_ERR_NULL_POINTER;
    if (int rc = check_rows(grad_rows, grad_row_stride, nr_positions, nr_levels, nr_feat)) return rc;
    if ((table.values && !table_aligned(table, nr_feat)) || !aligned8(lattice_values_grad)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (!positions_grad)
        return table_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, scale_factor, random_shift,
                              anneal_window, grad_rows, grad_row_stride, nullptr, lattice_values_grad, nullptr, workspace,
                              workspace_bytes, st, touched);
    // The position gradient gathers level by level and reads its upstream gradient as [level][feature][n]:
    // that copy lives at the front of the workspace; the rest serves the scatter and then the partial sums.
    const size_t copy_bytes = static_cast<size_t>(nr_levels) * nr_feat * static_cast<size_t>(nr_positions) * sizeof(float);
    const uintptr_t base = (reinterpret_cast<uintptr_t>(workspace) + 255u) & ~uintptr_t{255};
    const size_t lost = base - reinterpret_cast<uintptr_t>(workspace);
    if (workspace == nullptr || workspace_bytes < lost + copy_bytes) return PENC_ERR_WORKSPACE_TOO_SMALL;
    float* level_major = reinterpret_cast<float*>(base);
    const size_t copy_span = (copy_bytes + 255u) & ~size_t{255};
    void* rest = workspace_bytes >= lost + copy_span + 256 ? reinterpret_cast<void*>(base + copy_span) : nullptr;
    const size_t rest_bytes = rest ? workspace_bytes - lost - copy_span : 0;
    if (lattice_values_grad) {
        // the scattering kernel reads every (point, level) pair of the rows anyway and leaves the copy behind
        if (int rc = table_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, scale_factor, random_shift,
                                    anneal_window, grad_rows, grad_row_stride, nullptr, lattice_values_grad, level_major,
                                    rest, rest_bytes, st, touched))
            return rc;
    } else {
        const int cols = nr_feat * nr_levels;
        if (cols > 255) return PENC_ERR_BAD_SIZE;
        if (int rc = transpose_rows(grad_rows, grad_row_stride, level_major, nr_positions, cols, st)) return rc;
    }
    return positions_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor,
                              random_shift, anneal_window, level_major, positions_grad, rest, rest_bytes, st);
}

int penc_backward_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                           const float* positions, const float* lattice_values, const float* scale_factor,
                           const float* random_shift, const float* anneal_window, const float* grad_rows,
                           int64_t grad_row_stride, float* lattice_values_grad, float* positions_grad,
                           void* workspace, size_t workspace_bytes, void* stream) {
    return backward_rowmajor_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                                  scale_factor, random_shift, anneal_window, grad_rows, grad_row_stride, lattice_values_grad,
                                  positions_grad, workspace, workspace_bytes, stream);
}

int penc_backward_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                       const float* positions, const void* lattice_values_half, int table_format,
                       const float* scale_factor, const float* random_shift, const float* anneal_window,
                       const float* grad, int64_t grad_row_stride, float* lattice_values_grad, float* positions_grad,
                       void* workspace, size_t workspace_bytes, void* stream) {
    if (table_format != PENC_TABLE_FP16 && table_format != PENC_TABLE_BF16) return PENC_ERR_UNSUPPORTED_TABLE_FORMAT;
    const TableRef table{lattice_values_half, table_format};
    if (grad_row_stride != 0)
        return backward_rowmajor_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor,
                                      random_shift, anneal_window, grad, grad_row_stride, lattice_values_grad, positions_grad,
                                      workspace, workspace_bytes, stream);
    return backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor, random_shift,
                         anneal_window, grad, lattice_values_grad, positions_grad, workspace, workspace_bytes, stream);
}

int penc_backward_table_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                 const float* positions, const float* scale_factor, const float* random_shift,
                                 const float* anneal_window, const float* grad_rows, int64_t grad_row_stride,
                                 float* lattice_values_grad, void* workspace, size_t workspace_bytes, void* stream) {
    if (!lattice_values_grad) return PENC_ERR_NULL_POINTER;
    return penc_backward_rowmajor(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, nullptr, scale_factor,
                                  random_shift, anneal_window, grad_rows, grad_row_stride, lattice_values_grad, nullptr,
                                  workspace, workspace_bytes, stream);
}

static int double_backward_impl(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                const float* positions, const TableRef& table, const float* scale_factor,
                                const float* random_shift, const float* anneal_window,
                                const float* double_positions_grad, const float* grad, int64_t grad_row_stride,
                                float* lattice_values_grad, float* grad_grad_sliced_values, int concat_points,
                                void* workspace, size_t workspace_bytes, void* stream, uint32_t* touched = nullptr) {
    const int extra = penc_extra_levels(pos_dim, nr_feat, concat_points);
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, extra)) return rc;
    if (!positions || !table.values || !scale_factor || !random_shift || !anneal_window ||
        !double_positions_grad || !grad)
        return PENC_ERR_NULL_POINTER;
    if (!lattice_values_grad && !grad_grad_sliced_values) return PENC_ERR_NULL_POINTER;
    if (!table_aligned(table, nr_feat) || !aligned8(lattice_values_grad)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (grad_grad_sliced_values) {
        const int per_thread = gather_levels_per_thread(pos_dim);
        const dim3 grid(tiles(nr_positions), (nr_levels + extra + per_thread - 1) / per_thread);
        PENC_DISPATCH_DFT(pos_dim, nr_feat, table.format,
                          hipLaunchKernelGGL((grad_grad_kernel<DD, FF, TT>), grid, dim3(kBlock), 0, st,
                                             static_cast<int>(nr_positions), nr_levels, nr_levels + extra, per_thread, static_cast<uint32_t>(capacity),
                                             mask_of(capacity), positions, static_cast<const TT*>(table.values), scale_factor,
                                             random_shift, anneal_window, double_positions_grad, grad_grad_sliced_values));
        if (int rc = check_launch()) return rc;
    }
    if (!lattice_values_grad) return PENC_OK;
    return table_backward(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, scale_factor, random_shift, anneal_window,
                          grad, grad_row_stride, double_positions_grad, lattice_values_grad, nullptr, workspace,
                          workspace_bytes, st, touched);
}

int penc_double_backward_from_positions(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels,
                                        int capacity, const float* positions,
                                        const float* lattice_values, const float* scale_factor,
                                        const float* random_shift, const float* anneal_window,
                                        const float* double_positions_grad,
                                        const float* grad_sliced_values, float* lattice_values_grad,
                                        float* grad_grad_sliced_values, int concat_points, void* workspace,
                                        size_t workspace_bytes, void* stream) {
    return double_backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                                scale_factor, random_shift, anneal_window, double_positions_grad, grad_sliced_values, 0,
                                lattice_values_grad, grad_grad_sliced_values, concat_points, workspace, workspace_bytes,
                                stream);
}

int penc_double_backward_from_positions_rowmajor(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels,
                                                 int capacity, const float* positions, const float* lattice_values,
                                                 const float* scale_factor, const float* random_shift,
                                                 const float* anneal_window, const float* double_positions_grad,
                                                 const float* grad_rows, int64_t grad_row_stride,
                                                 float* lattice_values_grad, float* grad_grad_sliced_values,
                                                 int concat_points, void* workspace, size_t workspace_bytes,
                                                 void* stream) {
    if (nr_levels > 0 && nr_positions > 0)
        if (int rc = check_rows(grad_rows, grad_row_stride, nr_positions, nr_levels, nr_feat)) return rc;
    return double_backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                                scale_factor, random_shift, anneal_window, double_positions_grad, grad_rows,
                                grad_row_stride, lattice_values_grad, grad_grad_sliced_values, concat_points, workspace,
                                workspace_bytes, stream);
}

int penc_double_backward_from_positions_half(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                             const float* positions, const void* lattice_values_half, int table_format,
                                             const float* scale_factor, const float* random_shift,
                                             const float* anneal_window, const float* double_positions_grad,
                                             const float* grad, int64_t grad_row_stride, float* lattice_values_grad,
                                             float* grad_grad_sliced_values, int concat_points, void* workspace,
                                             size_t workspace_bytes, void* stream) {
    if (table_format != PENC_TABLE_FP16 && table_format != PENC_TABLE_BF16) return PENC_ERR_UNSUPPORTED_TABLE_FORMAT;
    if (grad_row_stride != 0 && nr_levels > 0 && nr_positions > 0)
        if (int rc = check_rows(grad, grad_row_stride, nr_positions, nr_levels, nr_feat)) return rc;
    return double_backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions,
                                TableRef{lattice_values_half, table_format}, scale_factor, random_shift, anneal_window,
                                double_positions_grad, grad, grad_row_stride, lattice_values_grad, grad_grad_sliced_values,
                                concat_points, workspace, workspace_bytes, stream);
}

// The scalars of one AdamW step as torch.optim.AdamW forms them (in double), rounded once for the kernel.
static AdamWStep adamw_scalars(double lr, double beta1, double beta2, double eps, double weight_decay, int64_t step) {
    AdamWStep a;
    a.decay = static_cast<float>(1.0 - lr * weight_decay);
    a.one_minus_b1 = static_cast<float>(1.0 - beta1);
    a.b2 = static_cast<float>(beta2);
    a.one_minus_b2 = static_cast<float>(1.0 - beta2);
    a.step_size = static_cast<float>(lr / (1.0 - __builtin_pow(beta1, static_cast<double>(step))));
    a.inv_c2 = static_cast<float>(1.0 / __builtin_sqrt(1.0 - __builtin_pow(beta2, static_cast<double>(step))));
    a.eps = static_cast<float>(eps);
    return a;
}

int penc_adamw_step(float* params, const float* grads, float* exp_avg, float* exp_avg_sq, int64_t n, double lr,
                    double beta1, double beta2, double eps, double weight_decay, int64_t step, int skip_zero_gradients,
                    void* stream) {
    if (!params || !grads || !exp_avg || !exp_avg_sq) return PENC_ERR_NULL_POINTER;
    if (n <= 0 || step <= 0) return PENC_ERR_BAD_SIZE;
    const AdamWStep a = adamw_scalars(lr, beta1, beta2, eps, weight_decay, step);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uintptr_t all = reinterpret_cast<uintptr_t>(params) | reinterpret_cast<uintptr_t>(grads) |
                          reinterpret_cast<uintptr_t>(exp_avg) | reinterpret_cast<uintptr_t>(exp_avg_sq);
    const size_t count = static_cast<size_t>(n);
    const size_t vector_part = (all & 15u) == 0 ? count / 4 * 4 : 0;
    if (vector_part != 0) {
        const size_t blocks = (vector_part / 4 + kBlock - 1) / kBlock;
        if (blocks > 0x7FFFFFFFull) return PENC_ERR_BAD_SIZE;
        hipLaunchKernelGGL(adamw_step_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, st, params, grads,
                           exp_avg, exp_avg_sq, vector_part, a, skip_zero_gradients);
        if (int rc = check_launch()) return rc;
    }
    if (vector_part != count) {
        const size_t rest = count - vector_part;
        const size_t blocks = (rest + kBlock - 1) / kBlock;
        if (blocks > 0x7FFFFFFFull) return PENC_ERR_BAD_SIZE;
        hipLaunchKernelGGL(adamw_step_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(kBlock), 0, st,
                           params + vector_part, grads + vector_part, exp_avg + vector_part, exp_avg_sq + vector_part, rest, a,
                           skip_zero_gradients);
        if (int rc = check_launch()) return rc;
    }
    return PENC_OK;
}

size_t penc_touched_map_entries(int nr_feat, int nr_levels, int capacity) {
    if ((nr_feat != 2 && nr_feat != 4 && nr_feat != 8) || nr_levels <= 0 || capacity <= 0) return 0;
    return static_cast<size_t>(nr_levels) * (nr_feat / 2) * bins_for_capacity(capacity);
}

int penc_touched_range_slots(int capacity) { return capacity > 0 ? 1 << bin_shift_for_capacity(capacity) : 0; }

int penc_backward_sparse(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                         const float* positions, const float* lattice_values, const float* scale_factor,
                         const float* random_shift, const float* anneal_window, const float* grad, int64_t grad_row_stride,
                         float* lattice_values_grad, uint32_t* touched, float* positions_grad, void* workspace,
                         size_t workspace_bytes, void* stream) {
    if (!lattice_values_grad || !touched) return PENC_ERR_NULL_POINTER;
    const TableRef table{lattice_values, 0};
    if (grad_row_stride != 0)
        return backward_rowmajor_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor,
                                      random_shift, anneal_window, grad, grad_row_stride, lattice_values_grad, positions_grad,
                                      workspace, workspace_bytes, stream, touched);
    return backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, table, scale_factor, random_shift,
                         anneal_window, grad, lattice_values_grad, positions_grad, workspace, workspace_bytes, stream, touched);
}

int penc_double_backward_from_positions_sparse(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                                               const float* positions, const float* lattice_values,
                                               const float* scale_factor, const float* random_shift,
                                               const float* anneal_window, const float* double_positions_grad,
                                               const float* grad, int64_t grad_row_stride, float* lattice_values_grad,
                                               uint32_t* touched, float* grad_grad_sliced_values, int concat_points,
                                               void* workspace, size_t workspace_bytes, void* stream) {
    if (!lattice_values_grad || !touched) return PENC_ERR_NULL_POINTER;
    if (grad_row_stride != 0 && nr_levels > 0 && nr_positions > 0)
        if (int rc = check_rows(grad, grad_row_stride, nr_positions, nr_levels, nr_feat)) return rc;
    return double_backward_impl(pos_dim, nr_feat, nr_positions, nr_levels, capacity, positions, TableRef{lattice_values, 0},
                                scale_factor, random_shift, anneal_window, double_positions_grad, grad, grad_row_stride,
                                lattice_values_grad, grad_grad_sliced_values, concat_points, workspace, workspace_bytes, stream,
                                touched);
}

// The launch shared by penc_adamw_step_sparse and penc_clear_touched: one workgroup per (slot range, level).
static int launch_touched_ranges(bool update, float* params, float* grads, float* exp_avg, float* exp_avg_sq, int nr_feat,
                                 int nr_levels, int capacity, uint32_t* touched, const AdamWStep& a, int clear, void* stream) {
    if (!grads || !touched || (update && (!params || !exp_avg || !exp_avg_sq))) return PENC_ERR_NULL_POINTER;
    if ((nr_feat != 2 && nr_feat != 4 && nr_feat != 8)) return PENC_ERR_UNSUPPORTED_NR_FEAT;
    if (nr_levels <= 0 || nr_levels > 65535 || capacity <= 0) return PENC_ERR_BAD_SIZE;
    const uintptr_t all = reinterpret_cast<uintptr_t>(grads) |
                          (update ? reinterpret_cast<uintptr_t>(params) | reinterpret_cast<uintptr_t>(exp_avg) |
                                        reinterpret_cast<uintptr_t>(exp_avg_sq)
                                  : uintptr_t{0});
    if ((all & 7u) != 0) return PENC_ERR_MISALIGNED;
    const uint32_t n_ranges = bins_for_capacity(capacity), shift = bin_shift_for_capacity(capacity);
    // 16 bytes at a time where every level's first value is 16-byte aligned, else 8 (a slot of two features)
    const bool wide = (all & 15u) == 0 && (static_cast<int64_t>(capacity) * nr_feat) % 4 == 0;
    const dim3 grid(n_ranges, static_cast<unsigned>(nr_levels));
    hipStream_t st = static_cast<hipStream_t>(stream);
#define PENC_LAUNCH_TOUCHED(UPDATE, VEC)                                                                                   \
    hipLaunchKernelGGL((touched_ranges_kernel<UPDATE, VEC>), grid, dim3(kBlock), 0, st, params, grads, exp_avg, exp_avg_sq, \
                       static_cast<uint32_t>(capacity), static_cast<uint32_t>(nr_feat), n_ranges, shift, touched, a, clear)
    if (update && wide) PENC_LAUNCH_TOUCHED(true, float4);
    else if (update) PENC_LAUNCH_TOUCHED(true, float2);
    else if (wide) PENC_LAUNCH_TOUCHED(false, float4);
    else PENC_LAUNCH_TOUCHED(false, float2);
#undef PENC_LAUNCH_TOUCHED
    return check_launch();
}

int penc_adamw_step_sparse(float* params, float* grads, float* exp_avg, float* exp_avg_sq, int nr_feat, int nr_levels,
                           int capacity, uint32_t* touched, double lr, double beta1, double beta2, double eps,
                           double weight_decay, int64_t step, int clear, void* stream) {
    if (step <= 0) return PENC_ERR_BAD_SIZE;
    return launch_touched_ranges(true, params, grads, exp_avg, exp_avg_sq, nr_feat, nr_levels, capacity, touched,
                                 adamw_scalars(lr, beta1, beta2, eps, weight_decay, step), clear, stream);
}

int penc_clear_touched(float* grads, int nr_feat, int nr_levels, int capacity, uint32_t* touched, void* stream) {
    return launch_touched_ranges(false, nullptr, grads, nullptr, nullptr, nr_feat, nr_levels, capacity, touched, AdamWStep{}, 1,
                                 stream);
}

int penc_transpose(const float* src, float* dst, int64_t rows, int cols, void* stream) {
    if (!src || !dst) return PENC_ERR_NULL_POINTER;
    if (rows <= 0 || cols <= 0 || cols > 255 || rows > ((int64_t{1} << 31) - 1) / cols) return PENC_ERR_BAD_SIZE;
    return transpose_rows(src, cols, dst, rows, cols, static_cast<hipStream_t>(stream));
}

int penc_simplex_debug(int pos_dim, int64_t nr_positions, int nr_levels, int capacity,
                       const float* positions, const float* scale_factor, const float* random_shift,
                       int gather_path, int* rem0, int* rank, int* slot, float* barycentric, void* stream) {
    if (int rc = check_geometry(pos_dim, 2, nr_positions, nr_levels, capacity, 0)) return rc;
    if (nr_positions > ((int64_t{1} << 31) - 1) / (pos_dim + 1) / nr_levels) return PENC_ERR_BAD_SIZE;
    if (!positions || !scale_factor || !random_shift) return PENC_ERR_NULL_POINTER;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(tiles(nr_positions), nr_levels);
#define PENC_LAUNCH_DEBUG(VIA_LDS)                                                                                   \
    PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((simplex_debug_kernel<DD, VIA_LDS>), grid, dim3(kBlock), 0, st,       \
                                                static_cast<int>(nr_positions), static_cast<uint32_t>(capacity),     \
                                                mask_of(capacity), positions, scale_factor, random_shift, rem0, rank, \
                                                slot, barycentric))
    if (gather_path) {
        PENC_LAUNCH_DEBUG(true);
    } else {
        PENC_LAUNCH_DEBUG(false);
    }
#undef PENC_LAUNCH_DEBUG
    return check_launch();
}

}  // extern "C"
