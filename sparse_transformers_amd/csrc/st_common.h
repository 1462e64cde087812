// Shared device helpers for the gfx950 sparse-MLP kernels: 16-byte vector
// loads, element unpacking for fp32 / fp16 / bf16, wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include "../../include/sparse_mlp_amd.h"

// Timeline hook: a build that defines ST_TL(i) before including the kernel
// sources can record a timestamp at stage i of a kernel; the library build
// leaves it empty.
#ifndef ST_TL
#define ST_TL(i)
#endif

namespace st {

constexpr int kWave = 64;

struct f16_t { uint16_t bits; };   // tag types: storage is 2 bytes, maths is fp32
struct bf16_t { uint16_t bits; };

template <typename T> struct Elem;
template <> struct Elem<float>  { static constexpr int kVec = 4; static constexpr int kBytes = 4; };
template <> struct Elem<f16_t>  { static constexpr int kVec = 8; static constexpr int kBytes = 2; };
template <> struct Elem<bf16_t> { static constexpr int kVec = 8; static constexpr int kBytes = 2; };

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));

// One 16-byte chunk of a row -> kVec floats.
template <typename T> __device__ __forceinline__ void unpack(const uint4 &v, float *f);

template <> __device__ __forceinline__ void unpack<float>(const uint4 &v, float *f)
{
    f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
    f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}
template <> __device__ __forceinline__ void unpack<f16_t>(const uint4 &v, float *f)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        half2_t h = __builtin_bit_cast(half2_t, w[i]);
        f[2 * i] = (float)h.x;
        f[2 * i + 1] = (float)h.y;
    }
}
template <> __device__ __forceinline__ void unpack<bf16_t>(const uint4 &v, float *f)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = __uint_as_float(w[i] << 16);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}

// One 32-bit word of a 2-byte type -> its two floats.
template <typename T> __device__ __forceinline__ void unpack_word(uint32_t w, float *f);
template <> __device__ __forceinline__ void unpack_word<f16_t>(uint32_t w, float *f)
{
    const half2_t h = __builtin_bit_cast(half2_t, w);
    f[0] = (float)h.x;
    f[1] = (float)h.y;
}
template <> __device__ __forceinline__ void unpack_word<bf16_t>(uint32_t w, float *f)
{
    f[0] = __uint_as_float(w << 16);
    f[1] = __uint_as_float(w & 0xffff0000u);
}

// float -> storage element (round to nearest even).
template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f)
{
    _Float16 h = (_Float16)f;
    f16_t r; r.bits = __builtin_bit_cast(uint16_t, h);
    return r;
}
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f)
{
    uint32_t u = __float_as_uint(f);
    bf16_t r;
    if ((u & 0x7fffffffu) > 0x7f800000u) { r.bits = (uint16_t)((u >> 16) | 0x40u); return r; }  // NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    r.bits = (uint16_t)(u >> 16);
    return r;
}

// pg += <g, x>, pu += <u, x> over one 16-byte chunk, elements in order.  Every kernel whose results are
// meant to agree bit for bit goes through this one function.  The 2-byte types use the two-element dot
// product instructions (fp32 accumulate) named explicitly: left to itself the compiler forms them from
// multiply-add chains in some places and not in others, and they round differently from the chain.
template <typename T>
__device__ __forceinline__ void dot_chunk(const uint4 &g, const uint4 &u, const uint4 &x, float &pg, float &pu)
{
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w}, xw[4] = {x.x, x.y, x.z, x.w};
    if constexpr (__is_same(T, float)) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            pg = fmaf(__uint_as_float(gw[e]), __uint_as_float(xw[e]), pg);
            pu = fmaf(__uint_as_float(uw[e]), __uint_as_float(xw[e]), pu);
        }
    } else if constexpr (__is_same(T, bf16_t)) {
        typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const bf16x2_t xv = __builtin_bit_cast(bf16x2_t, xw[j]);
            pg = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, gw[j]), xv, pg, false);
            pu = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, uw[j]), xv, pu, false);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t xv = __builtin_bit_cast(half2_t, xw[j]);
            pg = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, gw[j]), xv, pg, false);
            pu = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2_t, uw[j]), xv, pu, false);
        }
    }
}

// acc[e] += h * w[e] over one 16-byte chunk (same word-at-a-time scheme).
template <typename T> __device__ __forceinline__ void axpy_chunk(float h, const uint4 &w, float *acc)
{
    if constexpr (Elem<T>::kBytes == 4) {
        float fw[4];
        unpack<T>(w, fw);
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[e] = fmaf(h, fw[e], acc[e]);
    } else {
        const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float fw[2];
            unpack_word<T>(ww[j], fw);
            acc[2 * j] = fmaf(h, fw[0], acc[2 * j]);
            acc[2 * j + 1] = fmaf(h, fw[1], acc[2 * j + 1]);
        }
    }
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<f16_t>(f16_t v) { return (float)__builtin_bit_cast(_Float16, v.bits); }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return __uint_as_float((uint32_t)v.bits << 16); }

__device__ __forceinline__ uint4 ld16(const void *p) { return *reinterpret_cast<const uint4 *>(p); }
// Streaming variant for data that is read once per launch (weight rows): non-temporal hint.
__device__ __forceinline__ uint4 ld16_stream(const void *p)
{
    typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void *p, const uint4 &v) { *reinterpret_cast<uint4 *>(p) = v; }

// Sum over the 64 lanes of a wave with DPP row operations (no LDS traffic): four steps reduce each row of
// 16 lanes, the four row totals are then read through scalar registers.  Every lane receives the total.
template <int CTRL> __device__ __forceinline__ float dpp_add(float v)
{
    const int t = __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false);
    return v + __int_as_float(t);
}
__device__ __forceinline__ float wave_sum_dpp(float v)
{
    v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
    v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
    v = dpp_add<0x141>(v);  // row_half_mirror
    v = dpp_add<0x140>(v);  // row_mirror
    const int iv = __float_as_int(v);
    const float r0 = __int_as_float(__builtin_amdgcn_readlane(iv, 0));
    const float r1 = __int_as_float(__builtin_amdgcn_readlane(iv, 16));
    const float r2 = __int_as_float(__builtin_amdgcn_readlane(iv, 32));
    const float r3 = __int_as_float(__builtin_amdgcn_readlane(iv, 48));
    return (r0 + r1) + (r2 + r3);
}

// Sum over aligned groups of WIDTH lanes (4, 8, 16, 32 or 64); every lane of a group receives it.
template <int WIDTH> __device__ __forceinline__ float group_sum_dpp(float v)
{
    static_assert(WIDTH == 4 || WIDTH == 8 || WIDTH == 16 || WIDTH == 32 || WIDTH == 64, "unsupported group width");
    if constexpr (WIDTH == 64) {
        return wave_sum_dpp(v);
    } else {
        v = dpp_add<0xB1>(v);
        v = dpp_add<0x4E>(v);
        if constexpr (WIDTH >= 8) v = dpp_add<0x141>(v);
        if constexpr (WIDTH >= 16) v = dpp_add<0x140>(v);
        if constexpr (WIDTH == 32) v += __shfl_xor(v, 16, kWave);
        return v;
    }
}

__device__ __forceinline__ float activate(float v, int act)
{
    switch (act) {
    case ST_ACT_RELU: return v > 0.f ? v : 0.f;
    case ST_ACT_SILU: return v / (1.f + expf(-v));
    case ST_ACT_GELU_TANH: {
        const float k = 0.7978845608028654f;  // sqrt(2/pi)
        return 0.5f * v * (1.f + tanhf(k * (v + 0.044715f * v * v * v)));
    }
    case ST_ACT_SIGMOID: return 1.f / (1.f + expf(-v));
    default: return v;
    }
}

// The same with the hardware's exponential and reciprocal (about 1 ulp each, far inside what an fp16 / bf16
// result can show) where the exact forms cost an epilogue a microsecond: only for 16-bit outputs.
__device__ __forceinline__ float activate_fast(float v, int act)
{
    switch (act) {
    case ST_ACT_SILU: return v * __frcp_rn(1.f + __expf(-v));
    case ST_ACT_SIGMOID: return __frcp_rn(1.f + __expf(-v));
    default: return activate(v, act);
    }
}

// Host-side error plumbing shared by the C-ABI translation units.
void set_error(const char *fmt, ...);
int hip_fail(hipError_t e, const char *what);

#define ST_HIP(call)                                              \
    do {                                                          \
        hipError_t e__ = (call);                                  \
        if (e__ != hipSuccess) return ::st::hip_fail(e__, #call); \
    } while (0)

#define ST_REQUIRE(cond, ...)             \
    do {                                  \
        if (!(cond)) {                    \
            ::st::set_error(__VA_ARGS__); \
            return ST_ERR_ARG;            \
        }                                 \
    } while (0)

int device_cu_count();
// Lets `kernel` be launched with up to `bytes` of dynamic LDS (set once per kernel symbol).
int allow_dynamic_lds(const void *kernel, int bytes);

// Rows a thread group of the single-row decode kernels keeps in flight (18 16-byte loads per thread).
// The stand-alone and the fused kernel must agree on it: it decides which block sums which rows, and the
// two are meant to give the same bits.
template <typename T> struct DecodeRows { static constexpr int value = 6; };

// Blocks of the streaming decode kernels (one per CU by default) and the fixed-order sum of their
// fp32 partial rows [G][NB][H] into out[bcount][H].
int mlp_grid();
int launch_mlp_reduce(int dtype, const float *partials, int G, int NB, int bcount, int H, void *out,
                      hipStream_t stream);

// Rows of x from which st_mlp_forward switches from the streaming decode
// kernel to the MFMA kernels (fp16 / bf16 only).
constexpr int kPrefillMinRows = 32;
// 32 rows are two passes of the batch kernels, which beat the GEMM kernels at that size where they apply.
constexpr int kBatchMaxRows = 32;
int64_t prefill_workspace_bytes(int64_t M, int64_t H, int64_t n);
int launch_prefill(int dtype, const void *x, int M, int H, const void *gate, const void *up, const void *down, int n,
                   const int *n_dev, void *out, void *comb, long ldc, void *workspace, int act, int has_gate,
                   hipStream_t stream);

// MFMA kernels for a small batch of rows (batch_min_rows() <= B <= 32, fp16 / bf16, supported hidden sizes only).
int batch_min_rows();
bool batch_supported(int dtype, int H);
int64_t batch_workspace_bytes(int64_t H, int64_t n);
int launch_batch(int dtype, const void *x, int B, int H, const void *gate, const void *up, const void *down, int n,
                 const int *n_dev, void *out, void *comb, long ldc, void *workspace, int act, int has_gate,
                 hipStream_t stream);

// Double precision forward (plain kernels, for checking a model in fp64).
int64_t f64_workspace_bytes(int64_t B, int64_t H, int64_t n);
int launch_f64(const void *x, int B, int H, const void *gate, const void *up, const void *down, int n, const int *n_dev,
               void *out, void *comb, long ldc, void *workspace, int act, int has_gate, hipStream_t stream);

// Timing slot for one kernel launch; inert unless profiling is enabled.  ST_LAUNCH hands the slot's
// events to hipExtLaunchKernelGGL, which stamps them at the kernel's own begin and end (so the elapsed
// time is the kernel's execution time, without dispatch latency).
struct ProfScope {
    int slot;
    hipEvent_t start, stop;
    ProfScope(int kind, hipStream_t s);
};

#define ST_LAUNCH(ps, kern, grid, block, lds, stream, ...)                                              \
    do {                                                                                                \
        if ((ps).slot >= 0)                                                                             \
            hipExtLaunchKernelGGL(kern, grid, block, lds, stream, (ps).start, (ps).stop, 0, __VA_ARGS__); \
        else                                                                                            \
            hipLaunchKernelGGL(kern, grid, block, lds, stream, __VA_ARGS__);                             \
    } while (0)

}  // namespace st
