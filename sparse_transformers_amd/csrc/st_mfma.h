// Matrix-core helpers shared by the MFMA translation units (fp16 / bf16 16x16x32, fp32 accumulate).
//
// Operand layout of v_mfma_f32_16x16x32 on a 64-lane wave, D[m][n] += sum_k A[m][k] * B[k][n]:
//   A: lane l holds row m = l % 16, the 8 consecutive k of slice l / 16
//   B: lane l holds column n = l % 16, the 8 consecutive k of slice l / 16
//   D: lane l holds column n = l % 16, rows m = 4 * (l / 16) + e for e = 0..3
#pragma once

#include "st_common.h"

namespace st {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma;
template <> struct Mfma<f16_t> {
    static __device__ __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b),
                                                      c, 0, 0, 0);
    }
};
template <> struct Mfma<bf16_t> {
    static __device__ __forceinline__ f32x4_t run(const uint4 &a, const uint4 &b, f32x4_t c)
    {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};

__device__ __forceinline__ int device_count(int n_host, const int *n_dev)
{
    int n = n_host;
    if (n_dev) {
        const int nd = *n_dev;
        n = nd < n ? nd : n;
        if (n < 0) n = 0;
    }
    return n;
}

}  // namespace st
