// HIP kernels (gfx950, wave64) and C-ABI entry points of the permutohedral-lattice hash encoding.
//
// Work decomposition
//   forward, table backward, double backward : one thread per (point, level); blockIdx.y is the
//       level, so consecutive workgroups work on the same 8*capacity-byte slice of the table and
//       the level's scale factors / shifts / window weight are wave-uniform (scalar loads).
//   position backward : one thread per point, looping over the levels and summing in registers,
//       so the result is written once, without atomics and in a fixed order (the reference needs
//       D atomics per point-level because it gives each level its own block,
//       kernels/permutohedral_encoding/EncodingGPU.cuh:745-750).
//   A level whose anneal-window weight is exactly 0 contributes exactly 0 everywhere (for finite
//   table values), so such levels skip the table traffic and only store their zeros.
//
// Table gradient.  Thousands of points share a handful of lattice vertices at the coarse levels,
// so the scatter-add goes through two stages of combining before it reaches global fp32 atomics:
// a wave whose lanes all hit the same slot reduces with DPP and issues one atomic, and every
// workgroup accumulates into a small direct-mapped cache in LDS (tag = slot) that is flushed once
// at the end; a slot that loses its LDS line to another slot falls through to a global atomic, so
// the result does not depend on the cache ever hitting.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/penc.h"
#include "penc_lattice.hpp"

namespace penc {

constexpr int kBlock = 256;         // 4 wavefronts
constexpr int kCacheLines = 2048;   // LDS accumulate-cache lines per workgroup (tag + 2 floats = 24 KiB)
constexpr int kTilesPerGroup = 16;  // point tiles a table-gradient workgroup walks before flushing

__device__ __forceinline__ float2 load_vertex(const float* __restrict__ level_table, uint32_t slot) {
    return *reinterpret_cast<const float2*>(level_table + 2 * static_cast<size_t>(slot));
}

template <int D>
__device__ __forceinline__ fvec<D> load_point(const float* __restrict__ positions, int64_t n) {
    const float* p = positions + n * D;
    fvec<D> pos;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i); pos[i] = p[i]; });
    return pos;
}

// The D+1 table entries of a simplex, fetched back to back so that all loads are in flight together.
template <int D>
struct Vertices {
    fvec<D + 1> f0, f1;
};
template <int D>
__device__ __forceinline__ Vertices<D> load_vertices(const float* __restrict__ level_table, uvec<D + 1> h,
                                                     uint32_t capacity, uint32_t cap_mask) {
    Vertices<D> v;
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        const float2 x = load_vertex(level_table, to_slot(h[r], capacity, cap_mask));
        v.f0[r] = x.x;
        v.f1[r] = x.y;
    });
    return v;
}

// ------------------------------------------------------------------------------------------
// forward (EncodingGPU.cuh:68-256)

template <int D>
__global__ void __launch_bounds__(kBlock)
forward_kernel(int n_points, int n_levels, uint32_t capacity, uint32_t cap_mask,
               const float* __restrict__ positions, const float* __restrict__ table,
               const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
               const float* __restrict__ window, float* __restrict__ sliced, float points_scaling) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    const int level = blockIdx.y;
    float* out0 = sliced + (static_cast<size_t>(level) * 2) * n_points + n;
    float* out1 = out0 + n_points;

    if (level >= n_levels) {  // extra levels carrying the raw positions (:106-121)
        const int src = (level - n_levels) * 2;
        const float* p = positions + static_cast<size_t>(n) * D;
        *out0 = src < D ? p[src] * points_scaling : 0.0f;
        *out1 = src + 1 < D ? p[src + 1] * points_scaling : 0.0f;
        return;
    }
    const float w_level = window[level];
    if (w_level == 0.0f) {
        *out0 = 0.0f;
        *out1 = 0.0f;
        return;
    }
    const Located<D> s = locate<D>(load_point<D>(positions, n), random_shift + level * D, scale_factor + level * D);
    const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
    const Vertices<D> v = load_vertices<D>(table + static_cast<size_t>(level) * capacity * 2, h, capacity, cap_mask);
    const fvec<D + 1> w = barycentric<D>(s.rank, s.delta);
    float acc0 = 0.0f, acc1 = 0.0f;
    static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
        const float wr = w[r] * w_level;
        acc0 = acc0 + v.f0[r] * wr;
        acc1 = acc1 + v.f1[r] * wr;
    });
    *out0 = acc0;
    *out1 = acc1;
}

// ------------------------------------------------------------------------------------------
// scatter-add into the table gradient with wave- and workgroup-level combining

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

struct AccumCache {
    int tag[kCacheLines];
    float val[kCacheLines][2];
};

__device__ __forceinline__ void cache_clear(AccumCache& c) {
    for (int e = threadIdx.x; e < kCacheLines; e += kBlock) {
        c.tag[e] = -1;
        c.val[e][0] = 0.0f;
        c.val[e][1] = 0.0f;
    }
}

// Global fp32 atomics are serviced per 64-byte segment touched by a wave instruction, whatever
// the number of lanes in it (measured: 21 G segments/s, from 1 to 16 lanes per segment), so the two
// features of a slot, which are adjacent in memory, should leave in ONE instruction.  Lanes are
// paired (2p, 2p+1): first both lanes of a pair add the two features of the even lane's slot, then
// those of the odd lane's slot.  Must be called with all 64 lanes of the wave active.
__device__ __forceinline__ void global_add_pairs(float* __restrict__ level_grad, bool need, uint32_t slot,
                                                 float a0, float a1) {
    constexpr int kFromEven = 0xA0;  // quad_perm:[0,0,2,2]
    constexpr int kFromOdd = 0xF5;   // quad_perm:[1,1,3,3]
    const int odd = threadIdx.x & 1;
    const int slot_i = static_cast<int>(slot), need_i = need ? 1 : 0;
    const int a0_i = __builtin_bit_cast(int, a0), a1_i = __builtin_bit_cast(int, a1);
    {   // the even lane's contribution: even lane adds feature 0, odd lane feature 1
        const int s = __builtin_amdgcn_update_dpp(0, slot_i, kFromEven, 0xf, 0xf, true);
        const int n = __builtin_amdgcn_update_dpp(0, need_i, kFromEven, 0xf, 0xf, true);
        const int hi = __builtin_amdgcn_update_dpp(0, a1_i, kFromEven, 0xf, 0xf, true);
        const float v = __builtin_bit_cast(float, odd ? hi : a0_i);
        if (n) global_add(level_grad + 2 * static_cast<size_t>(static_cast<uint32_t>(s)) + odd, v);
    }
    {   // the odd lane's contribution
        const int s = __builtin_amdgcn_update_dpp(0, slot_i, kFromOdd, 0xf, 0xf, true);
        const int n = __builtin_amdgcn_update_dpp(0, need_i, kFromOdd, 0xf, 0xf, true);
        const int lo = __builtin_amdgcn_update_dpp(0, a0_i, kFromOdd, 0xf, 0xf, true);
        const float v = __builtin_bit_cast(float, odd ? a1_i : lo);
        if (n) global_add(level_grad + 2 * static_cast<size_t>(static_cast<uint32_t>(s)) + odd, v);
    }
}

// Adds (a0, a1) to slot `slot` of this level's gradient slice.  `active` is false for lanes that
// carry no point (tail of the last tile); they take part in the wave-wide steps only.
// Must be called with all 64 lanes of the wave active.
__device__ __forceinline__ void cache_add(AccumCache& c, float* __restrict__ level_grad, bool active,
                                          uint32_t slot, float a0, float a1) {
    // wave-uniform slot: one DPP reduction, one lane adds
    const uint32_t first = __builtin_amdgcn_readfirstlane(slot);
    if (__all(active && slot == first)) {
        a0 = wave_sum_to_last_lane(a0);
        a1 = wave_sum_to_last_lane(a1);
        active = (threadIdx.x & 63) == 63;
    }
    bool need_global = false;
    if (active) {
        const int e = static_cast<int>(slot & (kCacheLines - 1));
        int owner = c.tag[e];
        if (owner == -1) {
            owner = atomicCAS(&c.tag[e], -1, static_cast<int>(slot));
            if (owner == -1) owner = static_cast<int>(slot);
        }
        if (owner == static_cast<int>(slot)) {
            __hip_atomic_fetch_add(&c.val[e][0], a0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_fetch_add(&c.val[e][1], a1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        } else {
            need_global = true;
        }
    }
    global_add_pairs(level_grad, need_global, slot, a0, a1);
}

__device__ __forceinline__ void cache_flush(AccumCache& c, float* __restrict__ level_grad) {
    for (int e = threadIdx.x; e < kCacheLines; e += kBlock) {
        const int owner = c.tag[e];
        if (owner != -1) {
            float* g = level_grad + 2 * static_cast<size_t>(owner);
            global_add(g, c.val[e][0]);
            global_add(g + 1, c.val[e][1]);
        }
    }
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. the table (EncodingGPU.cuh:259-414)

template <int D>
__global__ void __launch_bounds__(kBlock)
backward_table_kernel(int n_points, uint32_t capacity, uint32_t cap_mask,
                      const float* __restrict__ positions, const float* __restrict__ scale_factor,
                      const float* __restrict__ random_shift, const float* __restrict__ window,
                      const float* __restrict__ grad_sliced, float* __restrict__ table_grad) {
    __shared__ AccumCache cache;
    const int level = blockIdx.y;
    const float w_level = window[level];
    if (w_level == 0.0f) return;
    cache_clear(cache);
    __syncthreads();
    float* level_grad = table_grad + static_cast<size_t>(level) * capacity * 2;
    const float* g0p = grad_sliced + (static_cast<size_t>(level) * 2) * n_points;
    const float* g1p = g0p + n_points;
    const int first_tile = blockIdx.x * kTilesPerGroup;
    for (int t = 0; t < kTilesPerGroup; ++t) {
        const int tile_base = (first_tile + t) * kBlock;
        if (tile_base >= n_points) break;
        const int n = tile_base + threadIdx.x;
        const bool active = n < n_points;
        const int nn = active ? n : n_points - 1;
        const float g0 = g0p[nn], g1 = g1p[nn];
        const Located<D> s = locate<D>(load_point<D>(positions, nn), random_shift + level * D, scale_factor + level * D);
        const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
        const fvec<D + 1> w = barycentric<D>(s.rank, s.delta);
        static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
            const float wr = w[r] * w_level;
            cache_add(cache, level_grad, active, to_slot(h[r], capacity, cap_mask), g0 * wr, g1 * wr);
        });
    }
    __syncthreads();
    cache_flush(cache, level_grad);
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. positions (EncodingGPU.cuh:530-769)

template <int D>
__global__ void __launch_bounds__(kBlock)
backward_pos_kernel(int n_points, int n_levels, uint32_t capacity, uint32_t cap_mask,
                    const float* __restrict__ positions, const float* __restrict__ table,
                    const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                    const float* __restrict__ window, const float* __restrict__ grad_sliced,
                    float* __restrict__ positions_grad) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    const fvec<D> pos = load_point<D>(positions, n);
    fvec<D> total = 0.0f;
    for (int level = 0; level < n_levels; ++level) {
        const float w_level = window[level];
        if (w_level == 0.0f) continue;
        const float* sf = scale_factor + level * D;
        const Located<D> s = locate<D>(pos, random_shift + level * D, sf);
        const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
        const Vertices<D> v = load_vertices<D>(table + static_cast<size_t>(level) * capacity * 2, h, capacity, cap_mask);
        const float* gp = grad_sliced + (static_cast<size_t>(level) * 2) * n_points + n;
        const float g0 = gp[0], g1 = gp[n_points];
        const fvec<D + 1> dB = (v.f0 * w_level) * g0 + (v.f1 * w_level) * g1;  // :688-689
        total += bary_grad_to_pos_grad<D>(s.rank, dB, sf);
    }
    float* o = positions_grad + static_cast<size_t>(n) * D;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i); o[i] = total[i]; });
}

// ------------------------------------------------------------------------------------------
// double backward from d(loss)/d(position gradient): both halves in one pass
// (EncodingGPU.cuh:1016-1257 scatter into the table gradient, 1260-1493 grad of grad_sliced)

template <int D, bool kTableGrad, bool kGradGrad>
__global__ void __launch_bounds__(kBlock)
double_backward_kernel(int n_points, int n_levels, uint32_t capacity, uint32_t cap_mask,
                       const float* __restrict__ positions, const float* __restrict__ table,
                       const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                       const float* __restrict__ window, const float* __restrict__ double_pos_grad,
                       const float* __restrict__ grad_sliced, float* __restrict__ table_grad,
                       float* __restrict__ grad_grad_sliced) {
    __shared__ AccumCache cache;
    const int level = blockIdx.y;
    const bool extra_level = level >= n_levels;  // concat levels: zeros (:1290-1295)
    const float w_level = extra_level ? 0.0f : window[level];
    const bool live = w_level != 0.0f;
    if (!live && !kGradGrad) return;
    if (kTableGrad && live) {
        cache_clear(cache);
        __syncthreads();
    }
    const int lvl = extra_level ? 0 : level;
    float* level_grad = kTableGrad ? table_grad + static_cast<size_t>(lvl) * capacity * 2 : nullptr;
    const float* level_table = table + static_cast<size_t>(lvl) * capacity * 2;
    const float* sf = scale_factor + lvl * D;
    const float* g0p = grad_sliced + (static_cast<size_t>(level) * 2) * n_points;
    const float* g1p = g0p + n_points;
    const int first_tile = blockIdx.x * kTilesPerGroup;
    for (int t = 0; t < kTilesPerGroup; ++t) {
        const int tile_base = (first_tile + t) * kBlock;
        if (tile_base >= n_points) break;
        const int n = tile_base + threadIdx.x;
        const bool active = n < n_points;
        const int nn = active ? n : n_points - 1;
        float gg0 = 0.0f, gg1 = 0.0f;
        if (live) {
            const Located<D> s = locate<D>(load_point<D>(positions, nn), random_shift + lvl * D, sf);
            const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
            Vertices<D> v;
            if constexpr (kGradGrad) v = load_vertices<D>(level_table, h, capacity, cap_mask);
            const fvec<D + 1> dB = pos_grad_grad_to_bary<D>(s.rank, load_point<D>(double_pos_grad, nn), sf);
            float g0 = 0.0f, g1 = 0.0f;
            if constexpr (kTableGrad) {
                g0 = g0p[nn];
                g1 = g1p[nn];
            }
            static_for<D + 1>(PENC_BODY(r) {
        PENC_INDEX(r);
                const float wr = dB[r] * w_level;
                if constexpr (kGradGrad) {
                    gg0 += wr * v.f0[r];
                    gg1 += wr * v.f1[r];
                }
                if constexpr (kTableGrad)
                    cache_add(cache, level_grad, active, to_slot(h[r], capacity, cap_mask), wr * g0, wr * g1);
            });
        }
        if (kGradGrad && active) {
            float* o = grad_grad_sliced + (static_cast<size_t>(level) * 2) * n_points + n;
            o[0] = gg0;
            o[n_points] = gg1;
        }
    }
    if (kTableGrad && live) {
        __syncthreads();
        cache_flush(cache, level_grad);
    }
}

// ------------------------------------------------------------------------------------------
// introspection

template <int D>
__global__ void __launch_bounds__(kBlock)
simplex_debug_kernel(int n_points, uint32_t capacity, uint32_t cap_mask, const float* __restrict__ positions,
                     const float* __restrict__ scale_factor, const float* __restrict__ random_shift,
                     int* __restrict__ rem0, int* __restrict__ rank, int* __restrict__ slot,
                     float* __restrict__ bary) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n >= n_points) return;
    const int level = blockIdx.y;
    const Located<D> s = locate<D>(load_point<D>(positions, n), random_shift + level * D, scale_factor + level * D);
    const uvec<D + 1> h = vertex_hashes<D>(s.rank, s.hash0);
    const fvec<D + 1> w = barycentric<D>(s.rank, s.delta);
    const size_t o = (static_cast<size_t>(level) * n_points + n) * (D + 1);
    static_for<D + 1>(PENC_BODY(i) {
        PENC_INDEX(i);
        if (rem0) rem0[o + i] = s.rem0[i];
        if (rank) rank[o + i] = s.rank[i];
        if (slot) slot[o + i] = static_cast<int>(to_slot(h[i], capacity, cap_mask));
        if (bary) bary[o + i] = w[i];
    });
}

__global__ void __launch_bounds__(kBlock) fill_zero_kernel(float2* __restrict__ p, size_t n2) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n2; i += stride)
        p[i] = make_float2(0.0f, 0.0f);
}

// ------------------------------------------------------------------------------------------
// host side

inline int check_launch() { return hipGetLastError() == hipSuccess ? PENC_OK : PENC_ERR_LAUNCH; }

inline uint32_t mask_of(int capacity) {
    const uint32_t c = static_cast<uint32_t>(capacity);
    return (c & (c - 1)) == 0 ? c - 1 : 0u;
}

inline int check_geometry(int pos_dim, int nr_feat, int64_t n, int levels, int capacity, int extra) {
    if (pos_dim < 2 || pos_dim > 8) return PENC_ERR_UNSUPPORTED_POS_DIM;
    if (nr_feat != 2) return PENC_ERR_UNSUPPORTED_NR_FEAT;
    if (n <= 0 || levels <= 0 || capacity <= 0) return PENC_ERR_BAD_SIZE;
    const int64_t lim = (int64_t{1} << 31) - 1;
    if (n > lim / (2 * (int64_t{levels} + extra)) || n > lim / pos_dim) return PENC_ERR_BAD_SIZE;
    if (int64_t{capacity} > lim / (2 * int64_t{levels})) return PENC_ERR_BAD_SIZE;
    if (levels + extra > 65535) return PENC_ERR_BAD_SIZE;
    return PENC_OK;
}

inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

// Clears the table gradient with a fill kernel (float2 granularity: the array is only guaranteed
// 8-byte alignment).  A kernel rather than hipMemsetAsync so that callers may capture the call in
// a HIP graph.
inline int clear_table_grad(float* g, int levels, int capacity, hipStream_t st) {
    const size_t n2 = static_cast<size_t>(levels) * capacity;
    const size_t want = (n2 + kBlock * 8 - 1) / (kBlock * 8);
    const unsigned blocks = static_cast<unsigned>(want < 8192 ? want : 8192);
    hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(kBlock), 0, st, reinterpret_cast<float2*>(g), n2);
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

inline unsigned tiles(int64_t n) { return static_cast<unsigned>((n + kBlock - 1) / kBlock); }
inline unsigned tile_groups(int64_t n) { return (tiles(n) + kTilesPerGroup - 1) / kTilesPerGroup; }

}  // namespace penc

using namespace penc;

extern "C" {

const char* penc_status_string(int status) {
    switch (status) {
        case PENC_OK: return "ok";
        case PENC_ERR_NULL_POINTER: return "a required pointer is NULL";
        case PENC_ERR_BAD_SIZE: return "nr_positions, nr_levels and capacity must be positive and every array must stay below 2^31 elements";
        case PENC_ERR_UNSUPPORTED_POS_DIM: return "pos_dim must be 2,3,4,5,6,7 or 8";
        case PENC_ERR_UNSUPPORTED_NR_FEAT: return "nr_feat_per_level must be 2 since other values are not implemented";
        case PENC_ERR_MISALIGNED: return "lattice_values and lattice_values_grad must be 8-byte aligned";
        case PENC_ERR_LAUNCH: return "the HIP runtime rejected a kernel launch";
        default: return "unknown status";
    }
}

int penc_extra_levels(int pos_dim, int nr_feat, int concat_points) {
    if (!concat_points || nr_feat <= 0) return 0;
    return (pos_dim + nr_feat - 1) / nr_feat;
}

int penc_scale_factors(int pos_dim, int nr_levels, const float* sigmas, float* scale_factor_out) {
    if (!sigmas || !scale_factor_out) return PENC_ERR_NULL_POINTER;
    if (pos_dim < 1 || nr_levels < 1) return PENC_ERR_BAD_SIZE;
    for (int l = 0; l < nr_levels; ++l)
        for (int i = 0; i < pos_dim; ++i) {
            const float numerator = static_cast<float>(1.0 / __builtin_sqrt(static_cast<double>((i + 1) * (i + 2))));
            scale_factor_out[l * pos_dim + i] = numerator / sigmas[l];
        }
    return PENC_OK;
}

int penc_forward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                 const float* positions, const float* lattice_values, const float* scale_factor,
                 const float* random_shift, const float* anneal_window, float* sliced_values,
                 int concat_points, float points_scaling, void* stream) {
    const int extra = penc_extra_levels(pos_dim, nr_feat, concat_points);
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, extra)) return rc;
    if (!positions || !lattice_values || !scale_factor || !random_shift || !anneal_window || !sliced_values)
        return PENC_ERR_NULL_POINTER;
    if (!aligned8(lattice_values)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(tiles(nr_positions), nr_levels + extra);
    PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((forward_kernel<DD>), grid, dim3(kBlock), 0, st,
                                                static_cast<int>(nr_positions), nr_levels,
                                                static_cast<uint32_t>(capacity), mask_of(capacity), positions,
                                                lattice_values, scale_factor, random_shift, anneal_window,
                                                sliced_values, points_scaling));
    return check_launch();
}

int penc_backward(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels, int capacity,
                  const float* positions, const float* lattice_values, const float* scale_factor,
                  const float* random_shift, const float* anneal_window,
                  const float* grad_sliced_values, float* lattice_values_grad, float* positions_grad,
                  void* stream) {
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, 0)) return rc;
    if (!positions || !scale_factor || !random_shift || !anneal_window || !grad_sliced_values)
        return PENC_ERR_NULL_POINTER;
    if (!lattice_values_grad && !positions_grad) return PENC_ERR_NULL_POINTER;
    if (positions_grad && !lattice_values) return PENC_ERR_NULL_POINTER;
    if ((lattice_values && !aligned8(lattice_values)) || !aligned8(lattice_values_grad)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n = static_cast<int>(nr_positions);
    const uint32_t cap = static_cast<uint32_t>(capacity), mask = mask_of(capacity);
    if (lattice_values_grad) {
        if (int rc = clear_table_grad(lattice_values_grad, nr_levels, capacity, st)) return rc;
        const dim3 grid(tile_groups(nr_positions), nr_levels);
        PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((backward_table_kernel<DD>), grid, dim3(kBlock), 0, st, n, cap, mask,
                                                    positions, scale_factor, random_shift, anneal_window,
                                                    grad_sliced_values, lattice_values_grad));
        if (int rc = check_launch()) return rc;
    }
    if (positions_grad) {
        PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((backward_pos_kernel<DD>), dim3(tiles(nr_positions)), dim3(kBlock), 0,
                                                    st, n, nr_levels, cap, mask, positions, lattice_values,
                                                    scale_factor, random_shift, anneal_window, grad_sliced_values,
                                                    positions_grad));
        if (int rc = check_launch()) return rc;
    }
    return PENC_OK;
}

int penc_double_backward_from_positions(int pos_dim, int nr_feat, int64_t nr_positions, int nr_levels,
                                        int capacity, const float* positions,
                                        const float* lattice_values, const float* scale_factor,
                                        const float* random_shift, const float* anneal_window,
                                        const float* double_positions_grad,
                                        const float* grad_sliced_values, float* lattice_values_grad,
                                        float* grad_grad_sliced_values, int concat_points, void* stream) {
    const int extra = penc_extra_levels(pos_dim, nr_feat, concat_points);
    if (int rc = check_geometry(pos_dim, nr_feat, nr_positions, nr_levels, capacity, extra)) return rc;
    if (!positions || !lattice_values || !scale_factor || !random_shift || !anneal_window ||
        !double_positions_grad || !grad_sliced_values)
        return PENC_ERR_NULL_POINTER;
    if (!lattice_values_grad && !grad_grad_sliced_values) return PENC_ERR_NULL_POINTER;
    if (!aligned8(lattice_values) || !aligned8(lattice_values_grad)) return PENC_ERR_MISALIGNED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n = static_cast<int>(nr_positions);
    const uint32_t cap = static_cast<uint32_t>(capacity), mask = mask_of(capacity);
    if (lattice_values_grad)
        if (int rc = clear_table_grad(lattice_values_grad, nr_levels, capacity, st)) return rc;
    const dim3 block(kBlock);
#define PENC_LAUNCH_DB(TG, GG, LEVELS)                                                                           \
    PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((double_backward_kernel<DD, TG, GG>),                            \
                                                dim3(tile_groups(nr_positions), LEVELS), block, 0, st, n, nr_levels, \
                                                cap, mask, positions, lattice_values, scale_factor, random_shift, \
                                                anneal_window, double_positions_grad, grad_sliced_values,        \
                                                lattice_values_grad, grad_grad_sliced_values))
    if (lattice_values_grad && grad_grad_sliced_values) {
        PENC_LAUNCH_DB(true, true, nr_levels + extra);
    } else if (lattice_values_grad) {
        PENC_LAUNCH_DB(true, false, nr_levels);
    } else {
        PENC_LAUNCH_DB(false, true, nr_levels + extra);
    }
#undef PENC_LAUNCH_DB
    return check_launch();
}

int penc_simplex_debug(int pos_dim, int64_t nr_positions, int nr_levels, int capacity,
                       const float* positions, const float* scale_factor, const float* random_shift,
                       int* rem0, int* rank, int* slot, float* barycentric, void* stream) {
    if (int rc = check_geometry(pos_dim, 2, nr_positions, nr_levels, capacity, 0)) return rc;
    if (nr_positions > ((int64_t{1} << 31) - 1) / (pos_dim + 1) / nr_levels) return PENC_ERR_BAD_SIZE;
    if (!positions || !scale_factor || !random_shift) return PENC_ERR_NULL_POINTER;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(tiles(nr_positions), nr_levels);
    PENC_DISPATCH_D(pos_dim, hipLaunchKernelGGL((simplex_debug_kernel<DD>), grid, dim3(kBlock), 0, st,
                                                static_cast<int>(nr_positions), static_cast<uint32_t>(capacity),
                                                mask_of(capacity), positions, scale_factor, random_shift, rem0, rank,
                                                slot, barycentric));
    return check_launch();
}

}  // extern "C"
