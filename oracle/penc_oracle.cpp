// CPU oracle for the permutohedral-lattice hash encoding.
//
// THIS FILE IS TEST INFRASTRUCTURE.  It restates, on the CPU, the algorithm of the reference's
// five live GPU kernels so that the HIP kernels can be checked against it and so that a CPU
// throughput figure can be reported next to the GPU one.  Nothing that ships (the Python
// package, the C-ABI library) may link, import or call it; only the tests, the smoke check and
// the CPU-baseline leg of the benchmark do.
//
// The reference is CUDA-only and has no CPU path, no tests and no golden vectors, so this is a
// restatement written from the reference's text, not a build of it.  What pins each function is
// listed next to it ("pinned by"); the checks themselves live in tests/test_oracle_*.py.
//
// Reference citations are to kernels/permutohedral_encoding/EncodingGPU.cuh unless a file is named.
//
// Arithmetic contract (identical in the HIP kernels, so that simplex choice and hashed slots are
// bit-identical): fp32 throughout, compiled with -ffp-contract=off, and exactly one fused
// multiply-add in the index-determining code: elevated[i] = fma(-i, cf, sm)  (":135", which the
// reference's compiler contracts by default).  Every other product in the index path is exact in
// fp32 for |elevated| < 2^24, so contraction elsewhere cannot change an index.
//
// The templates are instantiated for fp32 (the oracle of record for values) and for fp64 (used
// only by gradient checks: finite differences and adjoint identities need the head-room).
// Scatter-adds can be accumulated in fp64 (`*_acc64` outputs: the oracle of record for atomically
// summed gradients) and/or in fp32 with `omp atomic` (the timed CPU baseline).

#include <cmath>
#include <cstdint>
#include <cstddef>
#include <cstring>
#include <omp.h>

namespace {

constexpr uint32_t kHashMul = 2531011u;  // ":29"

template <typename R> inline R fused_mul_add(R a, R b, R c);
template <> inline float fused_mul_add<float>(float a, float b, float c) { return std::fmaf(a, b, c); }
template <> inline double fused_mul_add<double>(double a, double b, double c) { return std::fma(a, b, c); }

// ":22-32": k = 0; for each key coordinate: k += key; k *= 2531011  (wrapping uint32).
// Pinned by: known answers evaluated as the polynomial sum(key_i * M^(D-i)) mod 2^32 in Python ints.
template <int D>
inline uint32_t lattice_hash(const int* key) {
    uint32_t k = 0;
    for (int i = 0; i < D; ++i) {
        k += static_cast<uint32_t>(key[i]);
        k *= kHashMul;
    }
    return k;
}

// ":34-45": slot = hash % capacity, no collision resolution.
template <int D>
inline int lattice_slot(const int* key, int capacity) {
    return static_cast<int>(lattice_hash<D>(key) % static_cast<uint32_t>(capacity));
}

// Everything the kernels derive from one (point, level) before touching the table.
template <int D, typename R>
struct Simplex {
    R elevated[D + 1];
    int rem0[D + 1];
    int rank[D + 1];
    R bary[D + 2];
};

// ":130-186": elevate, round to the nearest remainder-0 lattice point, rank the residuals,
// wrap back onto the hyperplane.
// Pinned by: sum(elevated) = 0 and |elevated| = |pos+shift|/sigma (the embedding is a scaled
// isometry); after the wrap sum(rem0) = 0 and rank is a permutation; reconstruction identity
// sum_r bary[r] * vertex_r = elevated together with bary >= 0, sum(bary) = 1 (the enclosing
// Delaunay simplex of the A_d* lattice is unique for a generic point).
template <int D, typename R>
inline void locate_simplex(const R* pos, const R* shift, const R* sf, Simplex<D, R>& s) {
    constexpr int D1 = D + 1;
    R sm = 0;
    for (int i = D; i > 0; --i) {
        R cf = (pos[i - 1] + shift[i - 1]) * sf[i - 1];
        s.elevated[i] = fused_mul_add<R>(-static_cast<R>(i), cf, sm);  // sm - i*cf, one rounding
        sm += cf;
    }
    s.elevated[0] = sm;

    const R inv = static_cast<R>(1) / static_cast<R>(D1);
    int sum = 0;
    for (int i = 0; i <= D; ++i) {
        R v = s.elevated[i] * inv;
        R up = std::ceil(v) * static_cast<R>(D1);
        R down = std::floor(v) * static_cast<R>(D1);
        s.rem0[i] = (up - s.elevated[i] < s.elevated[i] - down) ? static_cast<int>(up) : static_cast<int>(down);
        sum += s.rem0[i];
    }
    sum /= D1;

    for (int i = 0; i <= D; ++i) s.rank[i] = 0;
    for (int i = 0; i < D; ++i) {
        R di = s.elevated[i] - static_cast<R>(s.rem0[i]);
        for (int j = i + 1; j <= D; ++j) {
            R dj = s.elevated[j] - static_cast<R>(s.rem0[j]);
            if (di < dj) s.rank[i]++; else s.rank[j]++;
        }
    }
    for (int i = 0; i <= D; ++i) {
        s.rank[i] += sum;
        if (s.rank[i] < 0) {
            s.rank[i] += D1;
            s.rem0[i] += D1;
        } else if (s.rank[i] > D) {
            s.rank[i] -= D1;
            s.rem0[i] -= D1;
        }
    }
}

// ":190-199": barycentric weights of the D+1 simplex vertices.
template <int D, typename R>
inline void barycentric(Simplex<D, R>& s) {
    constexpr int D1 = D + 1;
    const R inv = static_cast<R>(1) / static_cast<R>(D1);
    for (int k = 0; k <= D1; ++k) s.bary[k] = 0;
    for (int i = 0; i <= D; ++i) {
        R delta = (s.elevated[i] - static_cast<R>(s.rem0[i])) * inv;
        s.bary[D - s.rank[i]] += delta;
        s.bary[D1 - s.rank[i]] -= delta;
    }
    s.bary[0] += static_cast<R>(1) + s.bary[D1];
}

// ":216-220": first D coordinates of vertex `r` of the simplex (the last one is implied).
template <int D, typename R>
inline void vertex_key(const Simplex<D, R>& s, int r, int* key) {
    for (int i = 0; i < D; ++i) {
        key[i] = s.rem0[i] + r;
        if (s.rank[i] > D - r) key[i] -= (D + 1);
    }
}

// ":1187-1218": chain d(loss)/d(position gradient) -> elevated -> barycentric, shared by both
// halves of the double backward.
template <int D, typename R>
inline void double_backward_bary(const Simplex<D, R>& s, const R* q, const R* sf, R* dB /*[D+2]*/) {
    constexpr int D1 = D + 1;
    const R inv = static_cast<R>(1) / static_cast<R>(D1);
    R dE[D1];
    for (int j = 0; j <= D; ++j) dE[j] = 0;
    for (int i = 0; i < D; ++i) {
        R g = q[i] * sf[i];
        for (int j = 0; j <= i; ++j) dE[j] += g;
    }
    for (int i = 0; i < D; ++i) dE[i + 1] -= q[i] * sf[i] * static_cast<R>(i + 1);
    for (int k = 0; k <= D1; ++k) dB[k] = 0;
    for (int i = 0; i <= D; ++i) {
        dB[D - s.rank[i]] += dE[i] * inv;
        dB[D1 - s.rank[i]] -= dE[i] * inv;
    }
    dB[0] += dB[D1];
}

// The chain of double_backward_bary with every term replaced by its magnitude: an upper bound of
// the sum of |terms| behind each dB[k], the scale its rounding error is relative to.
template <int D, typename R, typename A>
inline void double_backward_bary_magnitude(const Simplex<D, R>& s, const R* q, const R* sf, A* mB /*[D+2]*/) {
    constexpr int D1 = D + 1;
    const A inv = static_cast<A>(1) / static_cast<A>(D1);
    A mE[D1];
    for (int j = 0; j <= D; ++j) mE[j] = 0;
    for (int i = 0; i < D; ++i) {
        const A g = std::fabs(static_cast<A>(q[i]) * static_cast<A>(sf[i]));
        for (int j = 0; j <= i; ++j) mE[j] += g;
        mE[i + 1] += g * static_cast<A>(i + 1);
    }
    for (int k = 0; k <= D1; ++k) mB[k] = 0;
    for (int i = 0; i <= D; ++i) {
        mB[D - s.rank[i]] += mE[i] * inv;
        mB[D1 - s.rank[i]] += mE[i] * inv;
    }
    mB[0] += mB[D1];
}

inline int extra_levels(int pos_dim, int nr_feat, int concat_points) {
    // src/Encoding.cu:71-74: ceil(pos_dim / val_dim) extra levels carry the raw positions
    return concat_points ? (pos_dim + nr_feat - 1) / nr_feat : 0;
}

// ------------------------------------------------------------------------------------------
// introspection: everything the preamble produces, per (level, point)

template <int D, typename R>
void simplex_dump(int64_t N, int L, int C, const R* pos, const R* sf, const R* shift,
                  R* elevated, int* rem0, int* rank, R* bary, int* slot, int* keys) {
    constexpr int D1 = D + 1;
    for (int l = 0; l < L; ++l) {
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            Simplex<D, R> s;
            locate_simplex<D, R>(pos + n * D, shift + l * D, sf + l * D, s);
            barycentric<D, R>(s);
            const int64_t o = (static_cast<int64_t>(l) * N + n) * D1;
            for (int i = 0; i <= D; ++i) {
                if (elevated) elevated[o + i] = s.elevated[i];
                if (rem0) rem0[o + i] = s.rem0[i];
                if (rank) rank[o + i] = s.rank[i];
                if (bary) bary[o + i] = s.bary[i];
            }
            for (int r = 0; r <= D; ++r) {
                int key[D1];
                vertex_key<D, R>(s, r, key);
                if (slot) slot[o + r] = lattice_slot<D>(key, C);
                if (keys) {
                    for (int i = 0; i < D; ++i) keys[(o + r) * D1 + i] = key[i];
                    // the implied coordinate, from the same rule as the others (":216-220")
                    int kd = s.rem0[D] + r;
                    if (s.rank[D] > D - r) kd -= D1;
                    keys[(o + r) * D1 + D] = kd;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// The four kernels below take the number of features per level, F, as an argument.  The reference
// instantiates F = 2 only (include/permutohedral_encoding/Encoding.cuh:139-143 rejects the rest, the
// other instantiations are commented out at src/Encoding.cu:362-363), and its kernels are written
// for val_dim = 2; F = 4 is the same algorithm with the feature loops two steps longer, and is
// pinned by the same identities (the pinning tests run for both values).
constexpr int kMaxFeat = 8;

// ------------------------------------------------------------------------------------------
// forward, ":99-254"
// Pinned by: reproduction of affine functions on a collision-free table, constant table ->
// window[l], one-hot table entry -> barycentric weight.

template <int D, typename R>
void forward(int64_t N, int L, int C, int F, const R* pos, const R* table, const R* sf, const R* shift,
             const R* window, R* out, int concat_points, R points_scaling) {
    constexpr int D1 = D + 1;
    const int extra = extra_levels(D, F, concat_points);
    for (int l = 0; l < L; ++l) {
        const R w_lvl = window[l];
        const R* tl = table + static_cast<int64_t>(l) * C * F;
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            Simplex<D, R> s;
            locate_simplex<D, R>(pos + n * D, shift + l * D, sf + l * D, s);
            barycentric<D, R>(s);
            R acc[kMaxFeat];
            for (int f = 0; f < F; ++f) acc[f] = 0;
            for (int r = 0; r <= D; ++r) {
                int key[D1];
                vertex_key<D, R>(s, r, key);
                const int64_t h = static_cast<int64_t>(F) * lattice_slot<D>(key, C);
                const R w = s.bary[r] * w_lvl;
                for (int f = 0; f < F; ++f) acc[f] = acc[f] + tl[h + f] * w;
            }
            for (int f = 0; f < F; ++f) out[(static_cast<int64_t>(l) * F + f) * N + n] = acc[f];
        }
    }
    for (int e = 0; e < extra; ++e) {  // ":106-121"
        for (int f = 0; f < F; ++f) {
            const int src = f + e * F;
            R* o = out + (static_cast<int64_t>(L + e) * F + f) * N;
#pragma omp parallel for schedule(static)
            for (int64_t n = 0; n < N; ++n) o[n] = (src < D) ? pos[n * D + src] * points_scaling : static_cast<R>(0);
        }
    }
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. the table, ":291-293, 385-414".  Output logical layout (L, C, F) (the
// reference fills (L, 2, C) and returns the permuted view, src/Encoding.cu:141,204).
// Pinned by: adjoint identity <forward(T), g> = <T, backward(g)>.

template <int D, typename R, typename A>
void backward_table(int64_t N, int L, int C, int F, const R* pos, const R* sf, const R* shift, const R* window,
                    const R* grad, R* tgrad, A* tgrad_acc, A* tgrad_abs) {
    constexpr int D1 = D + 1;
    for (int l = 0; l < L; ++l) {
        const R w_lvl = window[l];
        const int64_t base = static_cast<int64_t>(l) * C * F;
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            Simplex<D, R> s;
            locate_simplex<D, R>(pos + n * D, shift + l * D, sf + l * D, s);
            barycentric<D, R>(s);
            R g[kMaxFeat];
            for (int f = 0; f < F; ++f) g[f] = grad[(static_cast<int64_t>(l) * F + f) * N + n];
            for (int r = 0; r <= D; ++r) {
                int key[D1];
                vertex_key<D, R>(s, r, key);
                const int64_t h = base + static_cast<int64_t>(F) * lattice_slot<D>(key, C);
                const R w = s.bary[r] * w_lvl;
                for (int f = 0; f < F; ++f) {
                    const R t = g[f] * w;
                    if (tgrad) {
#pragma omp atomic
                        tgrad[h + f] += t;
                    }
                    if (tgrad_acc) {
#pragma omp atomic
                        tgrad_acc[h + f] += static_cast<A>(t);
                    }
                    if (tgrad_abs) {
#pragma omp atomic
                        tgrad_abs[h + f] += std::fabs(static_cast<A>(t));
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// backward w.r.t. positions, ":562-564, 651-749".  Output logical layout (N, D) (the reference
// fills (D, N) and returns the transpose, src/Encoding.cu:152,205).  Levels are summed in
// ascending order here; the reference sums them with atomics in no fixed order.
// Pinned by: finite differences of the fp64 forward inside a simplex (exact: the interpolant is
// piecewise linear).

template <int D, typename R, typename A>
void backward_pos(int64_t N, int L, int C, int F, const R* pos, const R* table, const R* sf, const R* shift,
                  const R* window, const R* grad, R* pgrad, A* pgrad_acc, A* pgrad_abs) {
    constexpr int D1 = D + 1;
    const R inv = static_cast<R>(1) / static_cast<R>(D1);
#pragma omp parallel for schedule(static)
    for (int64_t n = 0; n < N; ++n) {
        R sum[D];
        A sum_acc[D], sum_abs[D];
        for (int i = 0; i < D; ++i) { sum[i] = 0; sum_acc[i] = 0; sum_abs[i] = 0; }
        for (int l = 0; l < L; ++l) {
            const R w_lvl = window[l];
            const R* tl = table + static_cast<int64_t>(l) * C * F;
            const R* sfl = sf + l * D;
            Simplex<D, R> s;
            locate_simplex<D, R>(pos + n * D, shift + l * D, sfl, s);
            R g[kMaxFeat];
            for (int f = 0; f < F; ++f) g[f] = grad[(static_cast<int64_t>(l) * F + f) * N + n];
            R dB[D + 2];
            A mB[D + 2];  // the same chain with every term replaced by its magnitude (the scale rounding errors are relative to)
            for (int k = 0; k <= D1; ++k) { dB[k] = 0; mB[k] = 0; }
            for (int r = 0; r <= D; ++r) {
                int key[D1];
                vertex_key<D, R>(s, r, key);
                const int64_t h = static_cast<int64_t>(F) * lattice_slot<D>(key, C);
                for (int f = 0; f < F; ++f) {
                    dB[r] += tl[h + f] * w_lvl * g[f];
                    mB[r] += std::fabs(static_cast<A>(tl[h + f] * w_lvl * g[f]));
                }
            }
            dB[D1] += dB[0];  // ":698"
            mB[D1] = mB[0];
            R dE[D1];
            A mE[D1];
            for (int i = 0; i <= D; ++i) {
                dE[i] = 0;
                dE[i] += dB[D - s.rank[i]] * inv;
                dE[i] -= dB[D1 - s.rank[i]] * inv;
                mE[i] = (mB[D - s.rank[i]] + mB[D1 - s.rank[i]]) * static_cast<A>(inv);
            }
            for (int i = 0; i < D; ++i) {
                R dP = 0;
                A mP = 0;
                for (int j = 0; j <= i; ++j) dP += dE[j] * sfl[i];
                for (int j = 0; j <= i; ++j) mP += mE[j] * std::fabs(static_cast<A>(sfl[i]));
                dP -= dE[i + 1] * sfl[i] * static_cast<R>(i + 1);
                mP += mE[i + 1] * std::fabs(static_cast<A>(sfl[i])) * static_cast<A>(i + 1);
                sum[i] += dP;
                sum_acc[i] += static_cast<A>(dP);
                sum_abs[i] += mP;
            }
        }
        for (int i = 0; i < D; ++i) {
            if (pgrad) pgrad[n * D + i] = sum[i];
            if (pgrad_acc) pgrad_acc[n * D + i] = sum_acc[i];
            if (pgrad_abs) pgrad_abs[n * D + i] = sum_abs[i];
        }
    }
}

// ------------------------------------------------------------------------------------------
// double backward from d(loss)/d(position gradient), ":1141-1252" (table half) and
// ":1290-1295, 1385-1491" (grad-of-grad half).
// Pinned by: the position gradient is bilinear in (table, grad), giving two adjoint identities
// <q, posgrad(T,g)> = <ggs(q,T), g> = <tablegrad2(q,g), T>.

template <int D, typename R, typename A>
void double_backward(int64_t N, int L, int C, int F, const R* pos, const R* table, const R* sf, const R* shift,
                     const R* window, const R* q, const R* grad, R* tgrad, A* tgrad_acc, A* tgrad_abs,
                     R* ggs, A* ggs_abs, int concat_points) {
    constexpr int D1 = D + 1;
    const int extra = extra_levels(D, F, concat_points);
    for (int l = 0; l < L; ++l) {
        const R w_lvl = window[l];
        const int64_t base = static_cast<int64_t>(l) * C * F;
#pragma omp parallel for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            Simplex<D, R> s;
            locate_simplex<D, R>(pos + n * D, shift + l * D, sf + l * D, s);
            R dB[D + 2];
            double_backward_bary<D, R>(s, q + n * D, sf + l * D, dB);
            A mB[D + 2];
            if (ggs_abs) double_backward_bary_magnitude<D, R, A>(s, q + n * D, sf + l * D, mB);
            R g[kMaxFeat], gg[kMaxFeat];
            A ma[kMaxFeat];
            for (int f = 0; f < F; ++f) {
                g[f] = grad[(static_cast<int64_t>(l) * F + f) * N + n];
                gg[f] = 0;
                ma[f] = 0;
            }
            for (int r = 0; r <= D; ++r) {
                int key[D1];
                vertex_key<D, R>(s, r, key);
                const int64_t h = base + static_cast<int64_t>(F) * lattice_slot<D>(key, C);
                for (int f = 0; f < F; ++f) {
                    const R t = dB[r] * w_lvl * g[f];
                    if (tgrad) {
#pragma omp atomic
                        tgrad[h + f] += t;
                    }
                    if (tgrad_acc) {
#pragma omp atomic
                        tgrad_acc[h + f] += static_cast<A>(t);
                    }
                    if (tgrad_abs) {
#pragma omp atomic
                        tgrad_abs[h + f] += std::fabs(static_cast<A>(t));
                    }
                    if (ggs) gg[f] += dB[r] * w_lvl * table[h + f];
                    if (ggs_abs) ma[f] += mB[r] * std::fabs(static_cast<A>(w_lvl)) * std::fabs(static_cast<A>(table[h + f]));
                }
            }
            for (int f = 0; f < F; ++f) {
                if (ggs) ggs[(static_cast<int64_t>(l) * F + f) * N + n] = gg[f];
                if (ggs_abs) ggs_abs[(static_cast<int64_t>(l) * F + f) * N + n] = ma[f];
            }
        }
    }
    for (int64_t k = static_cast<int64_t>(L) * F * N; k < static_cast<int64_t>(L + extra) * F * N; ++k) {
        if (ggs) ggs[k] = 0;
        if (ggs_abs) ggs_abs[k] = 0;
    }
}

// include/permutohedral_encoding/Encoding.cuh:55-69.  The numerator is evaluated in fp64 and
// rounded to fp32 when it is stored in the tensor (":62"); the division of that fp32 tensor element
// by the fp32 sigma (":63") is ATen's tensor / host-scalar, which multiplies by the rounded fp32
// reciprocal of the scalar (its "a * (1/b)" path for a scalar second operand).
// Pinned by: closed form 1/(sqrt((i+1)(i+2)) * sigma) within 2 ulp (three fp32 roundings); the choice
// between this rule and a true division (1 ulp apart for a quarter of the entries) by a GPU test
// that evaluates the reference's two statements with torch itself.
void scale_factors(int D, int L, const float* sigmas, float* sf) {
    for (int l = 0; l < L; ++l)
        for (int i = 0; i < D; ++i) {
            const float num = static_cast<float>(1.0 / std::sqrt(static_cast<double>((i + 1) * (i + 2))));
            const float reciprocal = 1.0f / sigmas[l];
            sf[l * D + i] = num * reciprocal;
        }
}

#define DISPATCH_D(D_, CALL)                                       \
    switch (D_) {                                                  \
        case 2: { constexpr int DD = 2; CALL; } break;             \
        case 3: { constexpr int DD = 3; CALL; } break;             \
        case 4: { constexpr int DD = 4; CALL; } break;             \
        case 5: { constexpr int DD = 5; CALL; } break;             \
        case 6: { constexpr int DD = 6; CALL; } break;             \
        case 7: { constexpr int DD = 7; CALL; } break;             \
        case 8: { constexpr int DD = 8; CALL; } break;             \
        default: return 2;                                         \
    }

inline bool bad_sizes(int64_t N, int L, int C) { return N <= 0 || L <= 0 || C <= 0; }
inline bool bad_feat(int F) { return F < 1 || F > kMaxFeat; }

}  // namespace

extern "C" {

int penc_oracle_num_threads(void) { return omp_get_max_threads(); }

int penc_oracle_hash(int pos_dim, const int* key, uint32_t* out) {
    DISPATCH_D(pos_dim, *out = lattice_hash<DD>(key));
    return 0;
}

int penc_oracle_slot(int pos_dim, const int* key, int capacity, int* out) {
    if (capacity <= 0) return 1;
    DISPATCH_D(pos_dim, *out = lattice_slot<DD>(key, capacity));
    return 0;
}

int penc_oracle_scale_factors(int pos_dim, int nr_levels, const float* sigmas, float* sf) {
    if (pos_dim < 1 || nr_levels < 1) return 1;
    scale_factors(pos_dim, nr_levels, sigmas, sf);
    return 0;
}

int penc_oracle_simplex(int pos_dim, int64_t N, int L, int C, const float* pos, const float* sf,
                        const float* shift, float* elevated, int* rem0, int* rank, float* bary,
                        int* slot, int* keys) {
    if (bad_sizes(N, L, C)) return 1;
    DISPATCH_D(pos_dim, (simplex_dump<DD, float>(N, L, C, pos, sf, shift, elevated, rem0, rank, bary, slot, keys)));
    return 0;
}

int penc_oracle_simplex_f64(int pos_dim, int64_t N, int L, int C, const double* pos, const double* sf,
                            const double* shift, double* elevated, int* rem0, int* rank, double* bary,
                            int* slot, int* keys) {
    if (bad_sizes(N, L, C)) return 1;
    DISPATCH_D(pos_dim, (simplex_dump<DD, double>(N, L, C, pos, sf, shift, elevated, rem0, rank, bary, slot, keys)));
    return 0;
}

int penc_oracle_forward(int pos_dim, int64_t N, int L, int C, int F, const float* pos, const float* table,
                        const float* sf, const float* shift, const float* window, float* out,
                        int concat_points, float points_scaling) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (forward<DD, float>(N, L, C, F, pos, table, sf, shift, window, out, concat_points, points_scaling)));
    return 0;
}

int penc_oracle_forward_f64(int pos_dim, int64_t N, int L, int C, int F, const double* pos, const double* table,
                            const double* sf, const double* shift, const double* window, double* out,
                            int concat_points, double points_scaling) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (forward<DD, double>(N, L, C, F, pos, table, sf, shift, window, out, concat_points, points_scaling)));
    return 0;
}

// tgrad (fp32, omp-atomic), tgrad_acc64 and tgrad_abs64 (fp64 sums of the terms and of their
// magnitudes) are each optional (NULL) and are accumulated INTO: the caller zero-fills them.
int penc_oracle_backward_table(int pos_dim, int64_t N, int L, int C, int F, const float* pos, const float* sf,
                               const float* shift, const float* window, const float* grad,
                               float* tgrad, double* tgrad_acc64, double* tgrad_abs64) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (backward_table<DD, float, double>(N, L, C, F, pos, sf, shift, window, grad, tgrad, tgrad_acc64, tgrad_abs64)));
    return 0;
}

int penc_oracle_backward_table_f64(int pos_dim, int64_t N, int L, int C, int F, const double* pos, const double* sf,
                                   const double* shift, const double* window, const double* grad,
                                   double* tgrad) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (backward_table<DD, double, double>(N, L, C, F, pos, sf, shift, window, grad, tgrad, nullptr, nullptr)));
    return 0;
}

int penc_oracle_backward_pos(int pos_dim, int64_t N, int L, int C, int F, const float* pos, const float* table,
                             const float* sf, const float* shift, const float* window, const float* grad,
                             float* pgrad, double* pgrad_acc64, double* pgrad_abs64) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (backward_pos<DD, float, double>(N, L, C, F, pos, table, sf, shift, window, grad, pgrad, pgrad_acc64, pgrad_abs64)));
    return 0;
}

int penc_oracle_backward_pos_f64(int pos_dim, int64_t N, int L, int C, int F, const double* pos, const double* table,
                                 const double* sf, const double* shift, const double* window,
                                 const double* grad, double* pgrad) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (backward_pos<DD, double, double>(N, L, C, F, pos, table, sf, shift, window, grad, pgrad, nullptr, nullptr)));
    return 0;
}

int penc_oracle_double_backward(int pos_dim, int64_t N, int L, int C, int F, const float* pos, const float* table,
                                const float* sf, const float* shift, const float* window,
                                const float* double_pos_grad, const float* grad, float* tgrad,
                                double* tgrad_acc64, double* tgrad_abs64, float* ggs, double* ggs_abs64,
                                int concat_points) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (double_backward<DD, float, double>(N, L, C, F, pos, table, sf, shift, window, double_pos_grad, grad, tgrad, tgrad_acc64, tgrad_abs64, ggs, ggs_abs64, concat_points)));
    return 0;
}

int penc_oracle_double_backward_f64(int pos_dim, int64_t N, int L, int C, int F, const double* pos, const double* table,
                                    const double* sf, const double* shift, const double* window,
                                    const double* double_pos_grad, const double* grad, double* tgrad,
                                    double* ggs, int concat_points) {
    if (bad_sizes(N, L, C) || bad_feat(F)) return 1;
    DISPATCH_D(pos_dim, (double_backward<DD, double, double>(N, L, C, F, pos, table, sf, shift, window, double_pos_grad, grad, tgrad, nullptr, nullptr, ggs, nullptr, concat_points)));
    return 0;
}

}  // extern "C"
