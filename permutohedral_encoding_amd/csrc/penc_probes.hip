// Memory-system probes: the rooflines the encoding kernels are priced against are measured, on
// the same GPU and in the same run, with kernels that do nothing but the memory operation in
// question.  None of this has a counterpart in the reference.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/penc.h"  // status codes
#include "../../include/penc_probes.h"

namespace {

constexpr int kBlock = 256;

__global__ void __launch_bounds__(kBlock) copy_kernel(const float4* __restrict__ src, float4* __restrict__ dst, size_t n4) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n4; i += stride) dst[i] = src[i];
}

// Reads n4 16-byte elements and writes one value per workgroup: the streaming rate of a kernel that only reads.
__global__ void __launch_bounds__(kBlock) read_kernel(const float4* __restrict__ src, size_t n4, float* __restrict__ out) {
    const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
    float acc = 0.0f;
    for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n4; i += stride) {
        const float4 v = src[i];
        acc += (v.x + v.y) + (v.z + v.w);
    }
    if (acc == 12345.678f) out[blockIdx.x] = acc;  // keeps the loads alive; practically never taken
}

// `per_thread` independent 8-byte loads per thread, indices coalesced across the wave
// (idx[k][thread]), one 8-byte store: the access pattern of the forward pass without its arithmetic.
template <int K>
__global__ void __launch_bounds__(kBlock) gather_kernel(const float2* __restrict__ table, const int* __restrict__ idx,
                                                       size_t n_threads, float2* __restrict__ out) {
    const size_t t = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_threads) return;
    int slot[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot[k] = idx[k * n_threads + t];
    float2 v[K];
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = table[slot[k]];
    float2 acc = make_float2(0.0f, 0.0f);
#pragma unroll
    for (int k = 0; k < K; ++k) {
        acc.x += v[k].x;
        acc.y += v[k].y;
    }
    out[t] = acc;
}


// The same gathers with the knobs a kernel author could turn, so that the benchmark can show which
// setting this memory system serves fastest and price the encoding's gathers at that rate:
//   P    points per thread: K * P independent loads are in flight per lane before any is used
//   KIND how the load is issued: 0 an ordinary global load, 1 the compiler's non-temporal load,
//        2.. a raw buffer load whose cache-policy bits are (KIND - 2): bit 0 = sc0, bit 1 = nt, bit 4 = sc1
//   the workgroup size is a launch parameter (threads beyond n_threads / P return at once)
template <int K, int P, int KIND>
__global__ void gather_variant_kernel(const float2* __restrict__ table, uint32_t table_bytes, const int* __restrict__ idx,
                                      size_t n_threads, float2* __restrict__ out) {
    const size_t t0 = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x);
    const size_t n_lanes = n_threads / P;  // point p of a lane is thread p * n_lanes + lane: coalesced index reads and stores
    if (t0 >= n_lanes) return;
    int slot[P][K];
#pragma unroll
    for (int p = 0; p < P; ++p)
#pragma unroll
        for (int k = 0; k < K; ++k) slot[p][k] = idx[k * n_threads + p * n_lanes + t0];
    float2 v[P][K];
    if constexpr (KIND >= 2) {
        const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float2*>(table), 0, static_cast<int>(table_bytes), 0x00020000);
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int k = 0; k < K; ++k) {
                typedef uint32_t u2 __attribute__((ext_vector_type(2)));
                const u2 raw = __builtin_amdgcn_raw_buffer_load_b64(rsrc, slot[p][k] * 8, 0, KIND - 2);
                const uint32_t lo = raw.x, hi = raw.y;
                v[p][k] = make_float2(__builtin_bit_cast(float, lo), __builtin_bit_cast(float, hi));
            }
    } else {
#pragma unroll
        for (int p = 0; p < P; ++p)
#pragma unroll
            for (int k = 0; k < K; ++k) {
                if constexpr (KIND == 1) {
                    typedef float f2 __attribute__((ext_vector_type(2)));
                    const f2 x = __builtin_nontemporal_load(reinterpret_cast<const f2*>(table) + slot[p][k]);
                    v[p][k] = make_float2(x.x, x.y);
                } else {
                    v[p][k] = table[slot[p][k]];
                }
            }
    }
#pragma unroll
    for (int p = 0; p < P; ++p) {
        float2 acc = make_float2(0.0f, 0.0f);
#pragma unroll
        for (int k = 0; k < K; ++k) {
            acc.x += v[p][k].x;
            acc.y += v[p][k].y;
        }
        out[p * n_lanes + t0] = acc;
    }
}

template <int K>
__global__ void __launch_bounds__(kBlock) scatter_kernel(float* __restrict__ table, const int* __restrict__ idx,
                                                        size_t n_threads) {
    const size_t t = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x;
    if (t >= n_threads) return;
    int slot[K];
#pragma unroll
    for (int k = 0; k < K; ++k) slot[k] = idx[k * n_threads + t];
#pragma unroll
    for (int k = 0; k < K; ++k) {
        float* p = table + 2 * static_cast<size_t>(slot[k]);
        __hip_atomic_fetch_add(p, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __hip_atomic_fetch_add(p + 1, 1.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

inline int check_launch() { return hipGetLastError() == hipSuccess ? PENC_OK : PENC_ERR_LAUNCH; }

}  // namespace

extern "C" {

int penc_probe_copy(const float* src, float* dst, int64_t n_float4, void* stream) {
    if (!src || !dst) return PENC_ERR_NULL_POINTER;
    if (n_float4 <= 0) return PENC_ERR_BAD_SIZE;
    const int64_t want = (n_float4 + kBlock * 4 - 1) / (kBlock * 4);
    const unsigned blocks = static_cast<unsigned>(want < 16384 ? want : 16384);
    hipLaunchKernelGGL(copy_kernel, dim3(blocks), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const float4*>(src), reinterpret_cast<float4*>(dst), static_cast<size_t>(n_float4));
    return check_launch();
}

int penc_probe_read(const float* src, int64_t n_float4, float* out, void* stream) {
    if (!src || !out) return PENC_ERR_NULL_POINTER;
    if (n_float4 <= 0) return PENC_ERR_BAD_SIZE;
    const int64_t want = (n_float4 + kBlock * 4 - 1) / (kBlock * 4);
    const unsigned blocks = static_cast<unsigned>(want < 16384 ? want : 16384);
    hipLaunchKernelGGL(read_kernel, dim3(blocks), dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<const float4*>(src), static_cast<size_t>(n_float4), out);
    return check_launch();
}

#define PENC_PROBE_K(K_, ...)                                   \
    switch (K_) {                                               \
        case 1: { constexpr int KK = 1; __VA_ARGS__; } break;   \
        case 2: { constexpr int KK = 2; __VA_ARGS__; } break;   \
        case 3: { constexpr int KK = 3; __VA_ARGS__; } break;   \
        case 4: { constexpr int KK = 4; __VA_ARGS__; } break;   \
        case 5: { constexpr int KK = 5; __VA_ARGS__; } break;   \
        case 6: { constexpr int KK = 6; __VA_ARGS__; } break;   \
        case 7: { constexpr int KK = 7; __VA_ARGS__; } break;   \
        case 8: { constexpr int KK = 8; __VA_ARGS__; } break;   \
        case 9: { constexpr int KK = 9; __VA_ARGS__; } break;   \
        default: return PENC_ERR_BAD_SIZE;                      \
    }

int penc_probe_gather(const float* table, const int* idx, int64_t n_threads, int per_thread, float* out, void* stream) {
    if (!table || !idx || !out) return PENC_ERR_NULL_POINTER;
    if (n_threads <= 0) return PENC_ERR_BAD_SIZE;
    const dim3 grid(static_cast<unsigned>((n_threads + kBlock - 1) / kBlock));
    PENC_PROBE_K(per_thread, hipLaunchKernelGGL((gather_kernel<KK>), grid, dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                                                reinterpret_cast<const float2*>(table), idx, static_cast<size_t>(n_threads),
                                                reinterpret_cast<float2*>(out)));
    return check_launch();
}

#define PENC_PROBE_KIND(KIND_, ...)                                       \
    switch (KIND_) {                                                      \
        case 0: { constexpr int KIND = 0; __VA_ARGS__; } break;           \
        case 1: { constexpr int KIND = 1; __VA_ARGS__; } break;           \
        case 2: { constexpr int KIND = 2; __VA_ARGS__; } break;           \
        case 3: { constexpr int KIND = 3; __VA_ARGS__; } break;           \
        case 4: { constexpr int KIND = 4; __VA_ARGS__; } break;           \
        case 18: { constexpr int KIND = 18; __VA_ARGS__; } break;         \
        case 19: { constexpr int KIND = 19; __VA_ARGS__; } break;         \
        default: return PENC_ERR_BAD_SIZE;                                \
    }
#define PENC_PROBE_P(P_, ...)                                   \
    switch (P_) {                                               \
        case 1: { constexpr int PP = 1; __VA_ARGS__; } break;   \
        case 2: { constexpr int PP = 2; __VA_ARGS__; } break;   \
        case 4: { constexpr int PP = 4; __VA_ARGS__; } break;   \
        default: return PENC_ERR_BAD_SIZE;                      \
    }
#define PENC_PROBE_K3(K_, ...)                                  \
    switch (K_) {                                               \
        case 4: { constexpr int KK = 4; __VA_ARGS__; } break;   \
        case 5: { constexpr int KK = 5; __VA_ARGS__; } break;   \
        case 9: { constexpr int KK = 9; __VA_ARGS__; } break;   \
        default: return PENC_ERR_BAD_SIZE;                      \
    }

int penc_probe_gather_variant(const float* table, int64_t table_slots, const int* idx, int64_t n_threads, int per_thread,
                              int points_per_thread, int block_threads, int load_kind, float* out, void* stream) {
    if (!table || !idx || !out) return PENC_ERR_NULL_POINTER;
    if (n_threads <= 0 || table_slots <= 0 || table_slots > (int64_t{1} << 28) || n_threads % points_per_thread != 0 ||
        block_threads < 64 || block_threads > 1024 || block_threads % 64 != 0)
        return PENC_ERR_BAD_SIZE;
    const int64_t lanes = n_threads / points_per_thread;
    const dim3 grid(static_cast<unsigned>((lanes + block_threads - 1) / block_threads));
    PENC_PROBE_K3(per_thread, PENC_PROBE_P(points_per_thread, PENC_PROBE_KIND(load_kind,
        hipLaunchKernelGGL((gather_variant_kernel<KK, PP, KIND>), grid, dim3(block_threads), 0, static_cast<hipStream_t>(stream),
                           reinterpret_cast<const float2*>(table), static_cast<uint32_t>(table_slots * 8), idx,
                           static_cast<size_t>(n_threads), reinterpret_cast<float2*>(out)))));
    return check_launch();
}

int penc_probe_scatter(float* table, const int* idx, int64_t n_threads, int per_thread, void* stream) {
    if (!table || !idx) return PENC_ERR_NULL_POINTER;
    if (n_threads <= 0) return PENC_ERR_BAD_SIZE;
    const dim3 grid(static_cast<unsigned>((n_threads + kBlock - 1) / kBlock));
    PENC_PROBE_K(per_thread, hipLaunchKernelGGL((scatter_kernel<KK>), grid, dim3(kBlock), 0, static_cast<hipStream_t>(stream),
                                                table, idx, static_cast<size_t>(n_threads)));
    return check_launch();
}

}  // extern "C"
