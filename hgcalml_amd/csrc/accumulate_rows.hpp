// Device helpers shared by the neighbour-accumulation kernels (forward,
// separate gradients, fused gradient): vector loads/stores of VEC consecutive
// features, dense matrices seen through raw buffer descriptors, the
// wave-per-vertex tile mapping, divide-free slot decoding and the fixed
// cross-lane reduction of the weight gradient.
#pragma once

#include "hgc_common.hpp"

namespace hgc {
namespace acc {

template <int VEC>
struct FeatVec;
template <>
struct FeatVec<4> {
    using type = float4;
};
template <>
struct FeatVec<1> {
    using type = float;
};

template <int VEC>
__device__ __forceinline__ void load_vec(const float *p, float (&x)[VEC]) {
    if constexpr (VEC == 4) {
        const float4 v = *reinterpret_cast<const float4 *>(p);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else if constexpr (VEC == 2) {
        const float2 v = *reinterpret_cast<const float2 *>(p);
        x[0] = v.x; x[1] = v.y;
    } else {
        x[0] = *p;
    }
}

template <int VEC>
__device__ __forceinline__ void load_vec_i(const int *p, int (&x)[VEC]) {
    if constexpr (VEC == 4) {
        const int4 v = *reinterpret_cast<const int4 *>(p);
        x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
    } else if constexpr (VEC == 2) {
        const int2 v = *reinterpret_cast<const int2 *>(p);
        x[0] = v.x; x[1] = v.y;
    } else {
        x[0] = *p;
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec(float *p, const float (&x)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<float4 *>(p) = make_float4(x[0], x[1], x[2], x[3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<float2 *>(p) = make_float2(x[0], x[1]);
    } else {
        *p = x[0];
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec_i(int *p, const int (&x)[VEC]) {
    if constexpr (VEC == 4) {
        *reinterpret_cast<int4 *>(p) = make_int4(x[0], x[1], x[2], x[3]);
    } else if constexpr (VEC == 2) {
        *reinterpret_cast<int2 *>(p) = make_int2(x[0], x[1]);
    } else {
        *p = x[0];
    }
}

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// The same for data that is touched once (a vertex's own row, its result row): the
// non-temporal hint keeps such lines from pushing re-used rows out of L2.
template <int VEC>
__device__ __forceinline__ void load_vec_once(const float *p, float (&x)[VEC]) {
    static_assert(VEC == 1 || VEC == 2, "one or two features per lane");
    if constexpr (VEC == 2) {
        const f32x2 v = __builtin_nontemporal_load(reinterpret_cast<const f32x2 *>(p));
        x[0] = v.x; x[1] = v.y;
    } else {
        x[0] = __builtin_nontemporal_load(p);
    }
}

template <int VEC>
__device__ __forceinline__ void store_vec_once(float *p, const float (&x)[VEC]) {
    static_assert(VEC == 1 || VEC == 2 || VEC == 4, "one, two or four features per lane");
    if constexpr (VEC == 4) {
        f32x4 v;
        v.x = x[0]; v.y = x[1]; v.z = x[2]; v.w = x[3];
        __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(p));
    } else if constexpr (VEC == 2) {
        f32x2 v;
        v.x = x[0]; v.y = x[1];
        __builtin_nontemporal_store(v, reinterpret_cast<f32x2 *>(p));
    } else {
        __builtin_nontemporal_store(x[0], p);
    }
}

__device__ __forceinline__ void store_once(uint4 *p, const uint4 &x) {
    u32x4 v;
    v.x = x.x; v.y = x.y; v.z = x.z; v.w = x.w;
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4 *>(p));
}

__device__ __forceinline__ int wave_vertex() {
    const int tile = xcd_contiguous_block(blockIdx.x, gridDim.x);
    return __builtin_amdgcn_readfirstlane(tile * 4 + (int)(threadIdx.x >> 6));
}

// The vertex a wave works on when the caller gives a processing order (a
// permutation of the vertices, e.g. their order along a space-filling sort):
// waves that run at the same time then work on vertices that share neighbours,
// and the rows they gather are found in L2. Results do not depend on it.
// Returns n_vert for waves beyond the last vertex.
__device__ __forceinline__ int wave_vertex(const int *__restrict__ order, int n_vert) {
    const int i = wave_vertex();
    if (i >= n_vert) return n_vert;
    if (!order) return i;
    const int v = __builtin_amdgcn_readfirstlane(order[i]);
    return (uint32_t)v < (uint32_t)n_vert ? v : n_vert;
}

// A dense [rows, cols] matrix of 4-byte elements seen through a raw buffer
// descriptor (stride 0, num_records = size in bytes, gfx9 data format word).
struct RowMatrix {
    __amdgpu_buffer_rsrc_t rsrc;
    uint32_t row_bytes;
    __device__ __forceinline__ RowMatrix(const void *base, size_t rows, size_t cols)
        : rsrc(__builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)(uint32_t)(rows * cols * 4u),
                                                 0x00020000)),
          row_bytes((uint32_t)cols * 4u) {}

    // x[0..VEC) = M[row, col .. col+VEC) with col = lane_bytes/4 (+ col_bytes/4)
    template <int VEC>
    __device__ __forceinline__ void load(int row, uint32_t lane_bytes, uint32_t (&x)[VEC]) const {
        load_at<VEC>((uint32_t)row * row_bytes, lane_bytes, x);
    }
    // same with the (wave-uniform) byte offset of the row given directly
    // AUX: cache policy bits of the buffer instruction (2 = non-temporal)
    template <int VEC, int AUX = 0>
    __device__ __forceinline__ void load_at(uint32_t row_byte_offset, uint32_t lane_bytes, uint32_t (&x)[VEC]) const {
        const int soff = (int)row_byte_offset;
        if constexpr (VEC == 4) {
            const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)lane_bytes, soff, AUX);
            x[0] = v.x; x[1] = v.y; x[2] = v.z; x[3] = v.w;
        } else if constexpr (VEC == 2) {
            const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (int)lane_bytes, soff, AUX);
            x[0] = v.x; x[1] = v.y;
        } else {
            x[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_bytes, soff, AUX);
        }
    }
    template <int VEC, int AUX = 0>
    __device__ __forceinline__ void load_at(uint32_t row_byte_offset, uint32_t lane_bytes, float (&x)[VEC]) const {
        uint32_t r[VEC];
        load_at<VEC, AUX>(row_byte_offset, lane_bytes, r);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = __uint_as_float(r[e]);
    }
    template <int VEC>
    __device__ __forceinline__ void load(int row, uint32_t lane_bytes, float (&x)[VEC]) const {
        uint32_t r[VEC];
        load<VEC>(row, lane_bytes, r);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = __uint_as_float(r[e]);
    }
    template <int VEC>
    __device__ __forceinline__ void load(int row, uint32_t lane_bytes, int (&x)[VEC]) const {
        uint32_t r[VEC];
        load<VEC>(row, lane_bytes, r);
#pragma unroll
        for (int e = 0; e < VEC; ++e) x[e] = (int)r[e];
    }
};

// x / K for 0 <= x < 2^31 without an integer divide
struct FastDiv {
    uint32_t magic;  // 0: K is a power of two
    int shift;
};

__device__ __forceinline__ int fast_div(int x, const FastDiv d) {
    return d.magic == 0 ? (int)((uint32_t)x >> d.shift) : (int)(__umulhi((uint32_t)x, d.magic) >> d.shift);
}

// VEC arg-max slot bytes of row `row`, columns lane_col .. lane_col+VEC
template <int VEC>
__device__ __forceinline__ void load_slots(__amdgpu_buffer_rsrc_t rsrc, int row, uint32_t row_bytes, uint32_t lane_col,
                                           int (&x)[VEC]) {
    const int soff = (int)((uint32_t)row * row_bytes);
    uint32_t packed;
    if constexpr (VEC == 4) packed = __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_col, soff, 0);
    else if constexpr (VEC == 2) packed = __builtin_amdgcn_raw_buffer_load_b16(rsrc, (int)lane_col, soff, 0);
    else packed = __builtin_amdgcn_raw_buffer_load_b8(rsrc, (int)lane_col, soff, 0);
#pragma unroll
    for (int e = 0; e < VEC; ++e) x[e] = (int)((packed >> (8 * e)) & 255u);
}

// 32 partial sums per lane in, after the call lane L holds the sum over all 64
// lanes of value index (L & 31). Fixed butterfly: deterministic summation order.
__device__ __forceinline__ float transpose_reduce_32(float (&val)[32]) {
    const int lane = lane_id();
#pragma unroll
    for (int h = 16; h >= 1; h >>= 1) {
        const bool upper = (lane & h) != 0;
#pragma unroll
        for (int i = 0; i < h; ++i) {
            const float a = val[i], b = val[i + h];
            const float send = upper ? a : b;
            const float keep = upper ? b : a;
            val[i] = keep + __shfl_xor(send, h, kWave);
        }
    }
    return val[0] + __shfl_xor(val[0], 32, kWave);
}

inline bool is_pow2(int x) { return x > 0 && (x & (x - 1)) == 0; }

// features per lane of the wave-per-vertex kernels: all 64 lanes busy and
// every access naturally aligned
inline int wave_vec(int n_feat, uintptr_t align_or) {
    if (n_feat % 256 == 0 && (align_or & 15u) == 0) return 4;
    if (n_feat % 128 == 0 && (align_or & 7u) == 0) return 2;
    return 1;
}

inline FastDiv make_fast_div(int k) {
    FastDiv d;
    if (is_pow2(k)) {
        d.magic = 0;
        d.shift = 0;
        while ((1 << d.shift) < k) ++d.shift;
        return d;
    }
    int s = 0;
    while ((1ll << s) < k) ++s;  // ceil(log2 k) >= 2
    d.magic = (uint32_t)((1ull << (31 + s)) / (uint32_t)k + 1);
    d.shift = s - 1;
    return d;
}

}  // namespace acc
}  // namespace hgc
