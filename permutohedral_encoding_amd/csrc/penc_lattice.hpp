// Device-side geometry of the permutohedral lattice for gfx950: everything a kernel derives from
// one (point, level) pair before it touches the hash table.
//
// The arithmetic that decides WHICH simplex and WHICH table slots a point uses is written so that
// it rounds exactly like the CPU checker's: fp32, no implicit contraction (the translation unit is
// compiled with -ffp-contract=off) and one explicit fused multiply-add in the elevation
// (reference: kernels/permutohedral_encoding/EncodingGPU.cuh:130-138, which the reference's
// compiler contracts the same way).
//
// The small per-thread arrays (D+1 residuals, ranks, weights ...) are held in vector VALUES
// (ext_vector_type) indexed only by compile-time constants, and are passed between the helpers
// by value, so that they are registers by construction and never addressable memory.  The reference indexes its barycentric array with a run-time rank
// (EncodingGPU.cuh:195-196), which on a GPU forces the array into scratch memory; here the
// residuals are first put in rank order with compare/select chains, after which every index is
// a compile-time constant:
//
//     sorted[m]  = residual of the coordinate whose rank is m            (m = 0..D)
//     weight[0]  = sorted[D] + (1 - sorted[0])
//     weight[r]  = sorted[D-r] - sorted[D+1-r]                           (r = 1..D)
//
// which is term for term what the reference's "+= delta / -= delta" loop accumulates.
//
// The hash (EncodingGPU.cuh:22-32) is a polynomial in the key coordinates modulo 2^32,
//     h(key) = sum_i key[i] * M^(D-i),  M = 2531011,
// and vertex r of the simplex has key[i] = rem0[i] + r - (D+1)*[rank[i] > D-r]
// (EncodingGPU.cuh:216-220), so consecutive vertices differ by a constant minus one power:
//     h_0     = sum_i rem0[i] * M^(D-i)
//     h_{r+1} = h_r + sum_i M^(D-i) - (D+1) * M^(D-c),   c = the coordinate whose rank is D-r
// (no term when c is the implied last coordinate).  All of it is wrapping uint32 arithmetic, so
// the slots are bit-identical to evaluating the reference's loop per vertex, at D multiplies per
// point instead of D*(D+1).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <utility>

namespace penc {

// Per-thread short arrays as SSA vector values.  They are deliberately not C arrays: a helper
// that receives `const float (&a)[N]` is optimised on its own before it is inlined, and there the
// optimiser turns a compare/select chain over a[0..N-1] into ONE load from a run-time-selected
// address, which after inlining pins the caller's array in scratch memory or LDS.  A vector
// passed by value has no address, so element access stays extractelement/insertelement.
template <int N> using fvec = float __attribute__((ext_vector_type(N)));
template <int N> using ivec = int __attribute__((ext_vector_type(N)));
template <int N> using uvec = uint32_t __attribute__((ext_vector_type(N)));

// Compile-time loop: body(integral_constant<int, 0>) ... body(integral_constant<int, N-1>), so
// that every vector index below is a constant expression.
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& body, std::integer_sequence<int, Is...>) {
    (body(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& body) {
    static_for_impl(static_cast<F&&>(body), std::make_integer_sequence<int, N>{});
}
// Loop body as a lambda: `PENC_BODY(i) { PENC_INDEX(i); ... }` makes `i` a constant expression.
#define PENC_BODY(var) [&](auto var##_constant) __attribute__((always_inline))
#define PENC_INDEX(var) constexpr int var = decltype(var##_constant)::value

constexpr uint32_t kHashMul = 2531011u;

constexpr uint32_t hash_pow(int e) {
    uint32_t r = 1u;
    for (int k = 0; k < e; ++k) r *= kHashMul;
    return r;
}

template <int D>
constexpr uint32_t hash_pow_sum() {
    uint32_t s = 0u;
    for (int i = 0; i < D; ++i) s += hash_pow(D - i);
    return s;
}

// Increment of the raw hash from one simplex vertex to the next when coordinate C is the one
// that starts to wrap (C == D: the implied last coordinate, which is not hashed).
template <int D, int C>
constexpr uint32_t hash_step() {
    return C < D ? hash_pow_sum<D>() - static_cast<uint32_t>(D + 1) * hash_pow(D - C) : hash_pow_sum<D>();
}

// Reduces a raw 32-bit hash to a table slot (EncodingGPU.cuh:34-36).  `cap_mask` is capacity-1
// when the capacity is a power of two and 0 otherwise.
__device__ __forceinline__ uint32_t to_slot(uint32_t h, uint32_t capacity, uint32_t cap_mask) {
    return cap_mask ? (h & cap_mask) : (h % capacity);
}

template <int D>
struct Located {
    ivec<D + 1> rem0;    // remainder-0 lattice point, after the hyperplane wrap
    ivec<D + 1> rank;    // rank of each coordinate's residual, after the wrap (a permutation of 0..D)
    fvec<D + 1> delta;   // (elevated[i] - rem0[i]) / (D+1)
    uint32_t hash0;      // raw hash of vertex 0
};

// Elevate, round, rank, wrap (EncodingGPU.cuh:130-186) for one point at one level.
// `shift` and `sf` point at this level's D random shifts and D scale factors.
template <int D>
__device__ __forceinline__ Located<D> locate(fvec<D> pos, const float* __restrict__ shift,
                                             const float* __restrict__ sf) {
    constexpr int D1 = D + 1;
    constexpr float kInv = 1.0f / D1;
    fvec<D1> elevated;
    float sm = 0.0f;
    static_for<D>(PENC_BODY(k) {
        PENC_INDEX(k);
        constexpr int i = D - k;  // i = D .. 1
        const float cf = (pos[i - 1] + shift[i - 1]) * sf[i - 1];
        elevated[i] = __builtin_fmaf(-static_cast<float>(i), cf, sm);
        sm += cf;
    });
    elevated[0] = sm;

    // Round every coordinate to the nearer multiple of D+1, the lower one at a tie (:149-158).  The
    // upper candidate is formed as down + (D+1) instead of ceil(v)*(D+1): the two differ only when v
    // is an integer, where the reference's candidates coincide and the lower one is chosen here too.
    fvec<D1> resid;  // elevated - rounded: exact in fp32 (the two are within (D+1)/2 of each other)
    ivec<D1> rem0;
    int sum = 0;
    static_for<D1>(PENC_BODY(i) {
        PENC_INDEX(i);
        const float e = elevated[i];
        const float down = __builtin_floorf(e * kInv) * static_cast<float>(D1);
        const float up = down + static_cast<float>(D1);
        const float b = (up - e < e - down) ? up : down;
        rem0[i] = static_cast<int>(b);
        resid[i] = e - b;
        sum += static_cast<int>(b);
    });
    sum /= D1;

    ivec<D1> rank = 0;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i);
        static_for<D - i>(PENC_BODY(jj) {
        PENC_INDEX(jj);
            constexpr int j = i + 1 + jj;
            const int lt = resid[i] < resid[j] ? 1 : 0;
            rank[i] += lt;
            rank[j] += 1 - lt;
        });
    });

    // Wrap back onto the hyperplane (:173-186): a rank pushed outside 0..D by the coordinate sum comes
    // back by D+1 and takes its rem0 along.  `moved` is that multiple of D+1 (0 or +-(D+1)).  The
    // residual after the wrap, elevated - (rounded + moved), is one rounding of an exact difference
    // whichever way it is bracketed, so it is formed from the (exact) residual before the wrap.
    Located<D> o;
    uint32_t h = 0u;
    static_for<D1>(PENC_BODY(i) {
        PENC_INDEX(i);
        const int rk = rank[i] + sum;
        int wrapped_rank;
        if constexpr ((D1 & (D1 - 1)) == 0) {
            wrapped_rank = rk & (D1 - 1);  // rk is within D+1 of 0..D: reduction modulo a power of two
        } else {
            wrapped_rank = rk < 0 ? rk + D1 : (rk > D ? rk - D1 : rk);
        }
        const int moved = wrapped_rank - rk;
        o.rank[i] = wrapped_rank;
        const int r0 = rem0[i] + moved;
        o.rem0[i] = r0;
        o.delta[i] = (resid[i] - static_cast<float>(moved)) * kInv;
        if constexpr (i < D) h += static_cast<uint32_t>(r0) * hash_pow(D - i);
    });
    o.hash0 = h;
    return o;
}

// Per-coordinate values put in rank order: out[m] = in[c] where rank[c] == m.
template <int D>
__device__ __forceinline__ fvec<D + 1> by_rank(ivec<D + 1> rank, fvec<D + 1> in) {
    fvec<D + 1> out;
    static_for<D + 1>(PENC_BODY(m) {
        PENC_INDEX(m);
        float acc = in[0];
        static_for<D>(PENC_BODY(cc) {
        PENC_INDEX(cc);
            constexpr int c = cc + 1;
            const float x = in[c];
            acc = (rank[c] == m) ? x : acc;
        });
        out[m] = acc;
    });
    return out;
}

template <int D>
__device__ __forceinline__ fvec<D + 1> barycentric_of_sorted(fvec<D + 1> sorted) {
    fvec<D + 1> w;
    w[0] = sorted[D] + (1.0f + (0.0f - sorted[0]));
    static_for<D>(PENC_BODY(rr) {
        PENC_INDEX(rr);
        constexpr int r = rr + 1;
        w[r] = sorted[D - r] - sorted[D + 1 - r];
    });
    return w;
}

// Barycentric weights of the D+1 vertices (EncodingGPU.cuh:190-199).
template <int D>
__device__ __forceinline__ fvec<D + 1> barycentric(ivec<D + 1> rank, fvec<D + 1> delta) {
    return barycentric_of_sorted<D>(by_rank<D>(rank, delta));
}

// Raw hashes of the D+1 vertices (EncodingGPU.cuh:212-223), by the incremental rule above.
template <int D>
__device__ __forceinline__ uvec<D + 1> vertex_hashes(ivec<D + 1> rank, uint32_t hash0) {
    uvec<D + 1> h;
    h[0] = hash0;
    static_for<D>(PENC_BODY(r) {
        PENC_INDEX(r);
        // the coordinate of rank D-r starts to wrap between vertex r and vertex r+1
        uint32_t step = hash_step<D, 0>();
        static_for<D>(PENC_BODY(cc) {
        PENC_INDEX(cc);
            constexpr int c = cc + 1;
            step = (rank[c] == D - r) ? hash_step<D, c>() : step;
        });
        h[r + 1] = h[r] + step;
    });
    return h;
}

// The same two results (residuals in rank order, raw vertex hashes) through LDS instead of the
// D(D+1) compare-and-select chains above: every thread owns a column of D+1 eight-byte cells
// (`column` points at the thread's cell of row 0, rows are `stride` cells apart, so the lanes of a
// wave hit distinct banks), writes {delta[c], hash step of coordinate c} to row rank[c] and reads
// the rows back in order.  A thread only reads what it wrote itself: no barrier.
template <int D>
__device__ __forceinline__ void sort_by_rank_lds(uint2* column, uint32_t stride, ivec<D + 1> rank, fvec<D + 1> delta,
                                                 uint32_t hash0, fvec<D + 1>& sorted, uvec<D + 1>& hashes) {
    static_for<D + 1>(PENC_BODY(c) {
        PENC_INDEX(c);
        const float d = delta[c];
        uint2 cell;
        cell.x = __builtin_bit_cast(uint32_t, d);
        cell.y = hash_step<D, c>();
        // ranks of finite points are a permutation of 0..D; the clamp keeps a point with NaN or
        // overflowing coordinates inside its own column
        const int row = rank[c] < 0 ? 0 : (rank[c] > D ? D : rank[c]);
        column[static_cast<uint32_t>(row) * stride] = cell;
    });
    uvec<D + 1> step;
    static_for<D + 1>(PENC_BODY(m) {
        PENC_INDEX(m);
        const uint2 cell = column[m * stride];
        sorted[m] = __builtin_bit_cast(float, cell.x);
        step[m] = cell.y;
    });
    hashes[0] = hash0;
    static_for<D>(PENC_BODY(r) {
        PENC_INDEX(r);
        hashes[r + 1] = hashes[r] + step[D - r];  // the coordinate of rank D-r starts to wrap here
    });
}

// The three gradient chains below evaluate their sums in the same order, with the same
// intermediate roundings, as the reference's loops, so that every term a kernel adds is the same
// fp32 number the CPU checker computes; only the order of atomic accumulation can then differ.

// d(loss)/d(barycentric) -> d(loss)/d(position) for one level (EncodingGPU.cuh:698-740), in three
// steps.  dB[r] is the derivative w.r.t. the weight of vertex r.
// Step 1: dE[i] = dB[D-rank[i]]/(D+1) - dB[D+1-rank[i]]/(D+1), with dB[D+1] = dB[0] (the wrap-around
// term, :698), as a function of the rank m: diff[m] = dB[D-m]/(D+1) - dB[D+1-m]/(D+1).
template <int D>
__device__ __forceinline__ fvec<D + 1> bary_grad_by_rank(fvec<D + 1> dB) {
    constexpr int D1 = D + 1;
    constexpr float kInv = 1.0f / D1;
    const fvec<D1> scaled = dB * kInv;
    fvec<D1> diff;
    diff[0] = scaled[D] - scaled[0];
    static_for<D>(PENC_BODY(mm) {
        PENC_INDEX(mm);
        constexpr int m = mm + 1;
        diff[m] = scaled[D - m] - scaled[D1 - m];
    });
    return diff;
}

// Step 2: dE[i] = diff[rank[i]], by compare-and-select chains.
template <int D>
__device__ __forceinline__ fvec<D + 1> pick_by_rank(ivec<D + 1> rank, fvec<D + 1> diff) {
    fvec<D + 1> dE;
    static_for<D + 1>(PENC_BODY(i) {
        PENC_INDEX(i);
        float acc = diff[0];
        static_for<D>(PENC_BODY(mm) {
            PENC_INDEX(mm);
            constexpr int m = mm + 1;
            const float x = diff[m];
            acc = (rank[i] == m) ? x : acc;
        });
        dE[i] = acc;
    });
    return dE;
}

// Step 3: dP[i] = sum_{j<=i} dE[j]*sf[i] - dE[i+1]*sf[i]*(i+1)   (:729-740)
template <int D>
__device__ __forceinline__ fvec<D> elevated_grad_to_pos_grad(fvec<D + 1> dE, const float* __restrict__ sf) {
    fvec<D> dP;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i);
        float acc = dE[0] * sf[i];
        static_for<i>(PENC_BODY(jj) {
            PENC_INDEX(jj);
            acc += dE[jj + 1] * sf[i];
        });
        acc -= dE[i + 1] * sf[i] * static_cast<float>(i + 1);
        dP[i] = acc;
    });
    return dP;
}

template <int D>
__device__ __forceinline__ fvec<D> bary_grad_to_pos_grad(ivec<D + 1> rank, fvec<D + 1> dB,
                                                         const float* __restrict__ sf) {
    return elevated_grad_to_pos_grad<D>(pick_by_rank<D>(rank, bary_grad_by_rank<D>(dB)), sf);
}

// d(loss)/d(position gradient) -> derivative w.r.t. each vertex weight (EncodingGPU.cuh:1187-1218),
// in two steps with the permutation into rank order between them.
// Step 1: the derivative w.r.t. the elevated coordinates, already divided by D+1.
template <int D>
__device__ __forceinline__ fvec<D + 1> pos_grad_grad_to_elevated(fvec<D> q, const float* __restrict__ sf) {
    constexpr int D1 = D + 1;
    constexpr float kInv = 1.0f / D1;
    fvec<D> g;
    static_for<D>(PENC_BODY(i) {
        PENC_INDEX(i);
        g[i] = q[i] * sf[i];
    });
    // dE[j] = g[j] + g[j+1] + ... + g[D-1] (summed in ascending order, :1187-1194), then
    // dE[j] -= g[j-1]*j (:1196-1199)
    fvec<D1> dE;
    dE[D] = 0.0f;
    static_for<D>(PENC_BODY(j) {
        PENC_INDEX(j);
        float acc = g[j];
        static_for<D - 1 - j>(PENC_BODY(k) {
            PENC_INDEX(k);
            acc += g[j + 1 + k];
        });
        dE[j] = acc;
    });
    static_for<D>(PENC_BODY(jj) {
        PENC_INDEX(jj);
        constexpr int j = jj + 1;
        dE[j] -= g[j - 1] * static_cast<float>(j);
    });
    dE *= kInv;
    return dE;
}

// Step 2, from dE in rank order: dB[k] = sorted[D-k] - sorted[D+1-k]; dB[D+1] = -sorted[0] is folded
// into dB[0] (:1218).
template <int D>
__device__ __forceinline__ fvec<D + 1> sorted_elevated_grad_to_bary(fvec<D + 1> sorted) {
    constexpr int D1 = D + 1;
    fvec<D1> dB;
    dB[0] = sorted[D] + (0.0f - sorted[0]);
    static_for<D>(PENC_BODY(rr) {
        PENC_INDEX(rr);
        constexpr int r = rr + 1;
        dB[r] = sorted[D - r] - sorted[D1 - r];
    });
    return dB;
}

template <int D>
__device__ __forceinline__ fvec<D + 1> pos_grad_grad_to_bary(ivec<D + 1> rank, fvec<D> q,
                                                             const float* __restrict__ sf) {
    return sorted_elevated_grad_to_bary<D>(by_rank<D>(rank, pos_grad_grad_to_elevated<D>(q, sf)));
}

}  // namespace penc
