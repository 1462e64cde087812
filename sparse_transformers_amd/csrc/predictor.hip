// LoRA importance predictor -> threshold mask -> union over the batch rows.
//
//   kernel 1  t[b,k]   = <x[b,:], A[k,:]>            one wave per rank row k
//   kernel 2  s[b,i]   = <t[b,:], Bm[i,:]>           LPR lanes per row i
//             mask[i]  = any_b( s[b,i] >= thr )      written as one byte per i
//
// The rank-r intermediate stays in fp32.  Replaces FastLoRAProjection.forward
// (src/modeling_skip.py:52-53) and the "naive" branch + any(dim=0) of
// SkipDecoderLayer._compute_binary_mask (src/modeling_skip.py:204-207,214).
#include "st_common.h"

namespace st {

constexpr int kPredBTile = 8;

template <typename T>
__global__ __launch_bounds__(kWave) void predictor_down_kernel(const T *__restrict__ x, int B, int H,
                                                               const T *__restrict__ A, int r, float *__restrict__ t)
{
    constexpr int VEC = Elem<T>::kVec;
    const int k = blockIdx.x, lane = threadIdx.x;
    const int chunks = H / VEC;
    const T *row = A + (size_t)k * H;
    for (int b0 = 0; b0 < B; b0 += kPredBTile) {
        float acc[kPredBTile];
#pragma unroll
        for (int b = 0; b < kPredBTile; ++b) acc[b] = 0.f;
        for (int c = lane; c < chunks; c += kWave) {
            float fw[VEC];
            unpack<T>(ld16(row + (size_t)c * VEC), fw);
#pragma unroll
            for (int b = 0; b < kPredBTile; ++b) {
                if (b0 + b < B) {
                    float fx[VEC];
                    unpack<T>(ld16(x + (size_t)(b0 + b) * H + (size_t)c * VEC), fx);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[b] = fmaf(fw[e], fx[e], acc[b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < kPredBTile; ++b) {
            const float s = wave_sum(acc[b]);
            if (lane == 0 && b0 + b < B) t[(size_t)(b0 + b) * r + k] = s;
        }
    }
}

constexpr int kPredRowsPerWave = 16;

// lpr_log2: lanes that share one row of Bm (2^lpr_log2 >= r/VEC, capped at 64)
template <typename T>
__global__ __launch_bounds__(kWave) void predictor_up_mask_kernel(const float *__restrict__ t, int B, int r,
                                                                  const T *__restrict__ Bm, int I, float thr,
                                                                  int cmp_ge, int lpr_log2,
                                                                  float *__restrict__ scores,
                                                                  uint8_t *__restrict__ mask)
{
    constexpr int VEC = Elem<T>::kVec;
    extern __shared__ __align__(16) unsigned char smem[];
    float *ts = reinterpret_cast<float *>(smem);  // [B][r]
    const int lane = threadIdx.x;
    for (int i = lane; i < B * r; i += kWave) ts[i] = t[i];
    __syncthreads();

    const int chunks = r / VEC;
    const int LPR = 1 << lpr_log2, rpi = kWave >> lpr_log2;  // rows per iteration
    const int cl = lane & (LPR - 1), gidx = lane >> lpr_log2;
    const int tile = blockIdx.x * kPredRowsPerWave;

    for (int it = 0; it * rpi < kPredRowsPerWave; ++it) {
        const int row = tile + it * rpi + gidx;
        const bool row_ok = row < I && (it * rpi + gidx) < kPredRowsPerWave;
        bool any = false;
        for (int b0 = 0; b0 < B; b0 += kPredBTile) {
            float s[kPredBTile];
#pragma unroll
            for (int b = 0; b < kPredBTile; ++b) s[b] = 0.f;
            for (int c = cl; c < chunks; c += LPR) {
                float fw[VEC];
                const uint4 w = row_ok ? ld16(Bm + (size_t)row * r + (size_t)c * VEC) : make_uint4(0u, 0u, 0u, 0u);
                unpack<T>(w, fw);
#pragma unroll
                for (int b = 0; b < kPredBTile; ++b) {
                    if (b0 + b < B) {
                        const float *tp = ts + (size_t)(b0 + b) * r + c * VEC;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) s[b] = fmaf(fw[e], tp[e], s[b]);
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < kPredBTile; ++b) {
                if (b0 + b < B) {  // uniform across the wave
                    const float v = group_sum(s[b], LPR);
                    any = any || (cmp_ge ? (v >= thr) : (v > thr));
                    if (scores && cl == 0 && row_ok) scores[(size_t)(b0 + b) * I + row] = v;
                }
            }
        }
        if (cl == 0 && row_ok) mask[row] = any ? 1 : 0;
    }
}

template <typename T>
static int launch_predictor(const void *x, int B, int H, const void *A, int r, const void *Bm, int I, float thr,
                            int cmp_ge, float *t_ws, float *scores, uint8_t *mask, hipStream_t stream)
{
    constexpr int VEC = Elem<T>::kVec;
    hipLaunchKernelGGL(predictor_down_kernel<T>, dim3(r), dim3(kWave), 0, stream, static_cast<const T *>(x), B, H,
                       static_cast<const T *>(A), r, t_ws);
    ST_HIP(hipGetLastError());
    const int chunks = r / VEC;
    int lpr_log2 = 0;
    while ((1 << lpr_log2) < chunks && lpr_log2 < 6) ++lpr_log2;
    const size_t lds = (size_t)B * r * sizeof(float);
    hipLaunchKernelGGL(predictor_up_mask_kernel<T>, dim3((I + kPredRowsPerWave - 1) / kPredRowsPerWave), dim3(kWave),
                       lds, stream, t_ws, B, r, static_cast<const T *>(Bm), I, thr, cmp_ge, lpr_log2, scores, mask);
    ST_HIP(hipGetLastError());
    return ST_OK;
}

}  // namespace st

extern "C" int st_predictor_mask(const void *x, int64_t B, int64_t H, const void *A, int64_t r, const void *Bm,
                                 int64_t I, int dtype, float thr, int cmp_ge, float *t_ws, float *scores,
                                 uint8_t *mask, void *stream)
{
    using namespace st;
    ST_REQUIRE(x && A && Bm && t_ws && mask, "st_predictor_mask: null pointer");
    ST_REQUIRE(dtype >= ST_F32 && dtype <= ST_BF16, "st_predictor_mask: unknown dtype %d", dtype);
    const int esz = dtype == ST_F32 ? 4 : 2;
    ST_REQUIRE(B >= 1 && B <= 64, "st_predictor_mask: B=%lld out of range [1,64]", (long long)B);
    ST_REQUIRE(H >= 1 && (H * esz) % 16 == 0, "st_predictor_mask: H=%lld rows are not 16-byte multiples",
               (long long)H);
    ST_REQUIRE(r >= 1 && (r * esz) % 16 == 0, "st_predictor_mask: rank %lld rows are not 16-byte multiples",
               (long long)r);
    ST_REQUIRE(I >= 1 && I <= (1 << 24), "st_predictor_mask: I=%lld out of range", (long long)I);
    ST_REQUIRE(B * r * 4 <= 64 * 1024, "st_predictor_mask: B*r=%lld too large for the LDS staging buffer",
               (long long)(B * r));
    const uintptr_t align = (uintptr_t)x | (uintptr_t)A | (uintptr_t)Bm;
    ST_REQUIRE((align & 15) == 0, "st_predictor_mask: pointers must be 16-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case ST_F32: return launch_predictor<float>(x, (int)B, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, scores, mask, s);
    case ST_F16: return launch_predictor<f16_t>(x, (int)B, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, scores, mask, s);
    default: return launch_predictor<bf16_t>(x, (int)B, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, scores, mask, s);
    }
}
