// Shared by the kernels of the link scorer that run their products on the matrix cores: the 16-byte operand chunks per
// element type, the tile geometry and the base-2 helpers.
#pragma once
#include "common.hip.h"

namespace pcfgnat {
namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int PT = 32;        // parents per tile
constexpr int LF_NT = 256;    // threads per workgroup: four waves
constexpr float LF_THIN_SUM = 7.888609e-31f;  // 2^-100: below it a sum of probabilities may have lost terms to underflow

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

constexpr float LF_LOG2E = 1.4426950408889634f, LF_LN2 = 0.6931471805599453f;
constexpr float LF_FLOOR = -1e30f;  // stands for "no term yet" where -inf would give inf - inf
__device__ __forceinline__ float ex2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float lg2(float x) { return __builtin_amdgcn_logf(x); }

template <typename T>
struct Chunk;
template <>
struct Chunk<__half> {
    static constexpr int EPC = 8;  // elements per 16-byte chunk
    // acc += a (rows) x b (columns) over the 16 elements the two halves of the wave hold
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, floatx16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot(const uint4 &a, const uint4 &b, float acc) {
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a.x), __builtin_bit_cast(half2_t, b.x), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a.y), __builtin_bit_cast(half2_t, b.y), acc, false);
        acc = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a.z), __builtin_bit_cast(half2_t, b.z), acc, false);
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, a.w), __builtin_bit_cast(half2_t, b.w), acc, false);
    }
    // element f of a row stored as chunks
    static __device__ __forceinline__ float elem(const uint4 *row, int f) { return __half2float(reinterpret_cast<const __half *>(row)[f]); }
    static __device__ __forceinline__ __half cast(float v) { return __float2half(v); }
};
template <>
struct Chunk<float> {
    static constexpr int EPC = 4;
    static __device__ __forceinline__ void mma(const uint4 &a, const uint4 &b, floatx16 &acc) {
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.x), __uint_as_float(b.x), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.y), __uint_as_float(b.y), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.z), __uint_as_float(b.z), acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a.w), __uint_as_float(b.w), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ float dot(const uint4 &a, const uint4 &b, float acc) {
        acc = __builtin_fmaf(__uint_as_float(a.x), __uint_as_float(b.x), acc);
        acc = __builtin_fmaf(__uint_as_float(a.y), __uint_as_float(b.y), acc);
        acc = __builtin_fmaf(__uint_as_float(a.z), __uint_as_float(b.z), acc);
        return __builtin_fmaf(__uint_as_float(a.w), __uint_as_float(b.w), acc);
    }
    static __device__ __forceinline__ float elem(const uint4 *row, int f) { return reinterpret_cast<const float *>(row)[f]; }
    static __device__ __forceinline__ float cast(float v) { return v; }
};

// right child of accumulator r in lane half kb, relative to the tile: rows (r % 4) + 4 * kb + 8 * (r / 4)
__device__ __forceinline__ int acc_row(int r, int kb) { return (r & 3) + 4 * kb + 8 * (r >> 2); }

// head dimensions with 1, 2, 4 or 8 chunks per lane of one head's row
inline bool fused_head_dim_built(int dtype, int64_t F) {
    const int64_t unit = dtype == PCFGNAT_F16 ? 16 : 8;
    return F == unit || F == 2 * unit || F == 4 * unit || F == 8 * unit;
}

}  // namespace
}  // namespace pcfgnat
