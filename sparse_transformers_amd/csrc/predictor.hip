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
constexpr int kPredDownThreads = 256;
constexpr int kPredDownUnroll = 2;  // chunks per thread issued together

// One block per rank row k: all loads of the row (and of x) are issued before
// any arithmetic, so the kernel costs one memory round trip.
// BT = rows of x per pass (1 for single-row decode, so that nothing is requested twice).
template <typename T, int BT>
__global__ __launch_bounds__(kPredDownThreads) void predictor_down_kernel(const T *__restrict__ x, int B, int H,
                                                                          const T *__restrict__ A, int r,
                                                                          float *__restrict__ t, int round_storage)
{
    constexpr int VEC = Elem<T>::kVec;
    __shared__ float red[kPredDownThreads / kWave][BT];
    const int k = blockIdx.x, tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int chunks = H / VEC;
    const T *row = A + (size_t)k * H;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    for (int b0 = 0; b0 < B; b0 += BT) {
        float acc[BT];
#pragma unroll
        for (int b = 0; b < BT; ++b) acc[b] = 0.f;
        for (int c0 = 0; c0 < chunks; c0 += kPredDownThreads * kPredDownUnroll) {
            uint4 w[kPredDownUnroll];
#pragma unroll
            for (int u = 0; u < kPredDownUnroll; ++u) {
                const int c = c0 + u * kPredDownThreads + tid;
                w[u] = c < chunks ? ld16(row + (size_t)c * VEC) : zero4;
            }
            // x for every row of the tile is requested together (clamped row: the surplus sums are dropped)
            uint4 xv[BT][kPredDownUnroll];
#pragma unroll
            for (int b = 0; b < BT; ++b) {
                const int bb = b0 + b < B ? b0 + b : B - 1;
#pragma unroll
                for (int u = 0; u < kPredDownUnroll; ++u) {
                    const int c = c0 + u * kPredDownThreads + tid;
                    xv[b][u] = ld16(x + (size_t)bb * H + (size_t)(c < chunks ? c : 0) * VEC);
                }
            }
#pragma unroll
            for (int u = 0; u < kPredDownUnroll; ++u) {
                float fw[VEC];
                unpack<T>(w[u], fw);   // zeros past the row end
#pragma unroll
                for (int b = 0; b < BT; ++b) {
                    float fx[VEC];
                    unpack<T>(xv[b][u], fx);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[b] = fmaf(fw[e], fx[e], acc[b]);
                }
            }
        }
#pragma unroll
        for (int b = 0; b < BT; ++b) {
            const float s = wave_sum_dpp(acc[b]);
            if (lane == 0) red[wave][b] = s;
        }
        __syncthreads();
        if (tid < BT && b0 + tid < B) {
            float s = 0.f;
#pragma unroll
            for (int w2 = 0; w2 < kPredDownThreads / kWave; ++w2) s += red[w2][tid];
            // (round_storage: the rank-r intermediate as a module in the storage type would hand it on)
            t[(size_t)(b0 + tid) * r + k] = round_storage ? to_float<T>(from_float<T>(s)) : s;
        }
        __syncthreads();
    }
}

constexpr int kPredUpThreads = 256;   // (128-thread blocks measure the same)
// Rows of Bm a wave owns: as few as keep every lane busy for one pass (four rows of 16 chunks, two of 32 or
// 64).  More rows per wave mean fewer blocks, and the layer measures slower: 16 rows per wave (128 blocks at
// I = 8192) cost 1 us per layer against 4, and 4 against 2 cost 1.2 us at r = 256 and 0.7 us at r = 440.
constexpr int pred_rows_per_wave(int lpr) { return lpr >= 32 ? 2 : 4; }
constexpr int kPredUpBTile = 8;

// LPR lanes share one row of Bm (LPR >= r/VEC unless the row needs several
// passes); a wave owns RPW consecutive rows and issues the loads of all of them
// before the rank-r intermediate is staged in LDS.
template <typename T, int LPR, int RPW>
__global__ __launch_bounds__(kPredUpThreads) void predictor_up_mask_kernel(const float *__restrict__ t,
                                                                  const T *__restrict__ Bm,
                                                                  float *__restrict__ scores,
                                                                  uint8_t *__restrict__ mask, int B, int r, int I,
                                                                  float thr, int flags)
{
    // (13 dwords of arguments, all of them in scalar registers when the wave starts; the three switches share one)
    const int cmp_ge = flags & 1, round_storage = (flags >> 1) & 1, accumulate = (flags >> 2) & 1;
    constexpr int VEC = Elem<T>::kVec;
    constexpr int RPI = kWave / LPR;                                          // rows per iteration
    constexpr int NIT = RPW / RPI > 0 ? RPW / RPI : 1;  // iterations per tile
    extern __shared__ __align__(16) unsigned char smem[];
    float *ts = reinterpret_cast<float *>(smem);  // [B][r]
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int chunks = r / VEC;
    const int cl = lane & (LPR - 1), gidx = lane / LPR;
    const int tile = (blockIdx.x * (kPredUpThreads / kWave) + wave) * RPW;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    float s[NIT][kPredUpBTile];
    bool any[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) any[it] = false;

    for (int b0 = 0; b0 < B || b0 == 0; b0 += kPredUpBTile) {
#pragma unroll
        for (int it = 0; it < NIT; ++it)
#pragma unroll
            for (int b = 0; b < kPredUpBTile; ++b) s[it][b] = 0.f;
        for (int c = cl; c < chunks || c == cl; c += LPR) {  // one pass unless r/VEC > LPR
            uint4 w[NIT];
#pragma unroll
            for (int it = 0; it < NIT; ++it) {
                const int ro = it * RPI + gidx;
                const int row = tile + ro;
                w[it] = (c < chunks && ro < RPW && row < I) ? ld16(Bm + (size_t)row * r + (size_t)c * VEC)
                                                                        : zero4;
            }
            if (b0 == 0 && c == cl) {  // stage t after the row loads are in flight
                // 16-byte pieces, two per thread requested together: one memory round trip per 8 KB
                // (a scalar copy loop pays one round trip per 256 bytes)
                const float4 *t4 = reinterpret_cast<const float4 *>(t);
                float4 *ts4 = reinterpret_cast<float4 *>(ts);
                const int n4 = (B * r) >> 2;
                for (int i0 = 0; i0 < n4; i0 += kPredUpThreads * 2) {
                    float4 v[2];
#pragma unroll
                    for (int u = 0; u < 2; ++u) {
                        const int i = i0 + u * kPredUpThreads + tid;
                        v[u] = t4[i < n4 ? i : n4 - 1];
                    }
#pragma unroll
                    for (int u = 0; u < 2; ++u)   // unconditional: the staging buffer is padded to whole batches
                        ts4[i0 + u * kPredUpThreads + tid] = v[u];
                }
                __syncthreads();
            }
            if (c < chunks) {
#pragma unroll
                for (int it = 0; it < NIT; ++it) {
                    float fw[VEC];
                    unpack<T>(w[it], fw);
#pragma unroll
                    for (int b = 0; b < kPredUpBTile; ++b) {
                        if (b0 + b < B) {
                            const float *tp = ts + (size_t)(b0 + b) * r + c * VEC;
#pragma unroll
                            for (int e = 0; e < VEC; ++e) s[it][b] = fmaf(fw[e], tp[e], s[it][b]);
                        }
                    }
                }
            }
            if (c + LPR >= chunks) break;
        }
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
            const int ro = it * RPI + gidx;
            const int row = tile + ro;
            const bool row_ok = ro < RPW && row < I;
#pragma unroll
            for (int b = 0; b < kPredUpBTile; ++b) {
                if (b0 + b < B) {  // uniform across the wave
                    float v = group_sum_dpp<LPR>(s[it][b]);
                    if (round_storage) v = to_float<T>(from_float<T>(v));
                    any[it] = any[it] || (cmp_ge ? (v >= thr) : (v > thr));
                    if (scores && cl == 0 && row_ok) scores[(size_t)(b0 + b) * I + row] = v;
                }
            }
        }
        if (b0 + kPredUpBTile >= B) break;
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
        const int ro = it * RPI + gidx;
        const int row = tile + ro;
        // (accumulate: a later pass over more rows of x only ever switches bytes on)
        if (cl == 0 && ro < RPW && row < I && (any[it] || !accumulate)) mask[row] = any[it] ? 1 : 0;
    }
}

// Several rows of x (B > 1), rank rows of at most LPR chunks: a lane keeps its chunk of t for eight rows of x
// in registers and reuses it for the NITER rows of Bm it visits, so the LDS is read once per lane instead of
// once per (row of Bm, row of x) -- the first form of the kernel was bound by exactly those reads (32-byte
// strides, half the banks idle) and took 1.3 us per additional row of x at r = 256.  All NITER row loads of a
// wave are issued before anything else.
template <typename T, int LPR, int NITER>
__global__ __launch_bounds__(kPredUpThreads) void predictor_up_mask_rows_kernel(const float *__restrict__ t,
                                                                       const T *__restrict__ Bm,
                                                                       float *__restrict__ scores,
                                                                       uint8_t *__restrict__ mask, int B, int r, int I,
                                                                       float thr, int flags)
{
    const int cmp_ge = flags & 1, round_storage = (flags >> 1) & 1, accumulate = (flags >> 2) & 1;   // (as above)
    constexpr int VEC = Elem<T>::kVec;
    constexpr int RPI = kWave / LPR;   // rows per iteration
    extern __shared__ __align__(16) unsigned char smem[];
    float *ts = reinterpret_cast<float *>(smem);  // [B][r]
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int chunks = r / VEC;
    const int cl = lane & (LPR - 1), gidx = lane / LPR;
    const int tile = (blockIdx.x * (kPredUpThreads / kWave) + wave) * (RPI * NITER);
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    const bool has_chunk = cl < chunks;

    uint4 w[NITER];
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int row = tile + it * RPI + gidx;
        w[it] = ld16(Bm + (size_t)(row < I ? row : I - 1) * r + (size_t)(has_chunk ? cl : 0) * VEC);
        if (!has_chunk) w[it] = zero4;
    }
    {   // stage t: 16-byte pieces, two per thread requested together (the buffer is padded to whole batches)
        const float4 *t4 = reinterpret_cast<const float4 *>(t);
        float4 *ts4 = reinterpret_cast<float4 *>(ts);
        const int n4 = (B * r) >> 2;
        for (int i0 = 0; i0 < n4; i0 += kPredUpThreads * 2) {
            float4 v[2];
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int i = i0 + u * kPredUpThreads + tid;
                v[u] = t4[i < n4 ? i : n4 - 1];
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) ts4[i0 + u * kPredUpThreads + tid] = v[u];
        }
        __syncthreads();
    }
    unsigned any = 0u;   // bit per iteration
    for (int b0 = 0; b0 < B; b0 += kPredUpBTile) {
        float tr[kPredUpBTile][VEC];
#pragma unroll
        for (int b = 0; b < kPredUpBTile; ++b) {
            const float *tp = ts + (size_t)(b0 + b < B ? b0 + b : B - 1) * r + (has_chunk ? cl : 0) * VEC;
#pragma unroll
            for (int e = 0; e < VEC; e += 4) {
                const float4 q = *reinterpret_cast<const float4 *>(tp + e);
                tr[b][e] = q.x; tr[b][e + 1] = q.y; tr[b][e + 2] = q.z; tr[b][e + 3] = q.w;
            }
        }
#pragma unroll
        for (int it = 0; it < NITER; ++it) {
            const int row = tile + it * RPI + gidx;
            float fw[VEC];
            unpack<T>(w[it], fw);   // zeros in lanes without a chunk
#pragma unroll
            for (int b = 0; b < kPredUpBTile; ++b) {
                if (b0 + b < B) {   // uniform
                    float acc = 0.f;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc = fmaf(fw[e], tr[b][e], acc);
                    float v = group_sum_dpp<LPR>(acc);
                    if (round_storage) v = to_float<T>(from_float<T>(v));
                    if (cmp_ge ? (v >= thr) : (v > thr)) any |= 1u << it;
                    if (scores && cl == 0 && row < I) scores[(size_t)(b0 + b) * I + row] = v;
                }
            }
        }
    }
#pragma unroll
    for (int it = 0; it < NITER; ++it) {
        const int row = tile + it * RPI + gidx;
        if (cl == 0 && row < I && (((any >> it) & 1u) || !accumulate)) mask[row] = (any >> it) & 1u;
    }
}

template <typename T, int LPR, int RPW>
static void launch_up_rpw(ProfScope &ps, const float *t_ws, int B, int r, const void *Bm, int I, float thr, int cmp_ge,
                          float *scores, uint8_t *mask, int round_storage, int accumulate, hipStream_t stream)
{
    constexpr size_t batch = (size_t)kPredUpThreads * 2 * 16;   // the staging buffer is padded to whole batches
    const size_t lds = ((size_t)B * r * sizeof(float) + batch - 1) / batch * batch;
    constexpr int rows = RPW * (kPredUpThreads / kWave);
    ST_LAUNCH(ps, (predictor_up_mask_kernel<T, LPR, RPW>), dim3((I + rows - 1) / rows), dim3(kPredUpThreads), lds,
              stream, t_ws, static_cast<const T *>(Bm), scores, mask, B, r, I, thr,
              (cmp_ge ? 1 : 0) | (round_storage ? 2 : 0) | (accumulate ? 4 : 0));
}

template <typename T, int LPR>
static void launch_up(ProfScope &ps, const float *t_ws, int B, int r, const void *Bm, int I, float thr, int cmp_ge,
                      float *scores, uint8_t *mask, int round_storage, int accumulate, hipStream_t stream)
{
    constexpr int NITER = LPR >= 16 ? LPR / 16 : 1;   // about four rows of Bm per wave (measured against 1, 2 and 8 per lane)
    if (B > 1 && r / Elem<T>::kVec <= LPR) {
        constexpr size_t batch = (size_t)kPredUpThreads * 2 * 16;
        const size_t lds = ((size_t)B * r * sizeof(float) + batch - 1) / batch * batch;
        constexpr int rows = (kWave / LPR) * NITER * (kPredUpThreads / kWave);
        ST_LAUNCH(ps, (predictor_up_mask_rows_kernel<T, LPR, NITER>), dim3((I + rows - 1) / rows), dim3(kPredUpThreads),
                  lds, stream, t_ws, static_cast<const T *>(Bm), scores, mask, B, r, I, thr,
                  (cmp_ge ? 1 : 0) | (round_storage ? 2 : 0) | (accumulate ? 4 : 0));
        return;
    }
    launch_up_rpw<T, LPR, pred_rows_per_wave(LPR)>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage,
                                                   accumulate, stream);
}

template <typename T>
static int launch_predictor(const void *x, int B, int H, const void *A, int r, const void *Bm, int I, float thr,
                            int cmp_ge, float *t_ws, float *scores, uint8_t *mask, int round_storage, int accumulate,
                            hipStream_t stream)
{
    constexpr int VEC = Elem<T>::kVec;
    {
        ProfScope ps(ST_K_PRED_DOWN, stream);
        if (B == 1)
            ST_LAUNCH(ps, (predictor_down_kernel<T, 1>), dim3(r), dim3(kPredDownThreads), 0, stream,
                      static_cast<const T *>(x), B, H, static_cast<const T *>(A), r, t_ws, round_storage);
        else if (B <= kPredBTile)
            ST_LAUNCH(ps, (predictor_down_kernel<T, kPredBTile>), dim3(r), dim3(kPredDownThreads), 0, stream,
                      static_cast<const T *>(x), B, H, static_cast<const T *>(A), r, t_ws, round_storage);
        else   // 9 to 16 rows of x in one pass (one memory round trip instead of two)
            ST_LAUNCH(ps, (predictor_down_kernel<T, 2 * kPredBTile>), dim3(r), dim3(kPredDownThreads), 0, stream,
                      static_cast<const T *>(x), B, H, static_cast<const T *>(A), r, t_ws, round_storage);
    }
    ST_HIP(hipGetLastError());
    const int chunks = r / VEC;
    {
        ProfScope ps(ST_K_PRED_UP_MASK, stream);
        if (chunks <= 4) launch_up<T, 4>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage, accumulate, stream);
        else if (chunks <= 8) launch_up<T, 8>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage, accumulate, stream);
        else if (chunks <= 16) launch_up<T, 16>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage, accumulate, stream);
        else if (chunks <= 32) launch_up<T, 32>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage, accumulate, stream);
        else launch_up<T, 64>(ps, t_ws, B, r, Bm, I, thr, cmp_ge, scores, mask, round_storage, accumulate, stream);
    }
    ST_HIP(hipGetLastError());
    return ST_OK;
}

}  // namespace st

extern "C" int st_predictor_mask_ex(const void *x, int64_t B, int64_t H, const void *A, int64_t r, const void *Bm,
                                    int64_t I, int dtype, float thr, int cmp_ge, int flags, float *t_ws, float *scores,
                                    uint8_t *mask, void *stream)
{
    using namespace st;
    ST_REQUIRE(x && A && Bm && t_ws && mask, "st_predictor_mask_ex: null pointer");
    ST_REQUIRE(dtype >= ST_F32 && dtype <= ST_BF16, "st_predictor_mask_ex: unknown dtype %d", dtype);
    const int esz = dtype == ST_F32 ? 4 : 2;
    ST_REQUIRE(B >= 1 && B <= (1 << 20), "st_predictor_mask_ex: B=%lld out of range", (long long)B);
    ST_REQUIRE(H >= 1 && (H * esz) % 16 == 0, "st_predictor_mask_ex: H=%lld rows are not 16-byte multiples",
               (long long)H);
    ST_REQUIRE(r >= 1 && (r * esz) % 16 == 0, "st_predictor_mask_ex: rank %lld rows are not 16-byte multiples",
               (long long)r);
    ST_REQUIRE(I >= 1 && I <= (1 << 24), "st_predictor_mask_ex: I=%lld out of range", (long long)I);
    ST_REQUIRE(r * 4 <= 56 * 1024, "st_predictor_mask_ex: rank %lld too large for the LDS staging buffer", (long long)r);
    const uintptr_t align = (uintptr_t)x | (uintptr_t)A | (uintptr_t)Bm;
    ST_REQUIRE((align & 15) == 0, "st_predictor_mask_ex: pointers must be 16-byte aligned");
    ST_REQUIRE((flags & ~ST_PRED_ROUND_STORAGE) == 0, "st_predictor_mask_ex: unknown flags %d", flags);
    const int round_storage = (flags & ST_PRED_ROUND_STORAGE) && dtype != ST_F32 ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Rows of x per pass: what the staging buffer of the second kernel holds, 64 at most.  Further passes reuse
    // the front of t_ws (the launches are ordered on the stream) and only ever switch mask bytes on.
    int64_t per = (56 * 1024) / (r * 4);
    per = per > 64 ? 64 : per;
    for (int64_t b0 = 0; b0 < B; b0 += per) {
        const int bc = (int)(B - b0 < per ? B - b0 : per);
        const void *xp = static_cast<const unsigned char *>(x) + (size_t)b0 * H * esz;
        float *sp = scores ? scores + (size_t)b0 * I : nullptr;
        const int acc = b0 > 0 ? 1 : 0;
        int rc;
        switch (dtype) {
        case ST_F32: rc = launch_predictor<float>(xp, bc, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, sp, mask, round_storage, acc, s); break;
        case ST_F16: rc = launch_predictor<f16_t>(xp, bc, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, sp, mask, round_storage, acc, s); break;
        default: rc = launch_predictor<bf16_t>(xp, bc, (int)H, A, (int)r, Bm, (int)I, thr, cmp_ge, t_ws, sp, mask, round_storage, acc, s); break;
        }
        if (rc != ST_OK) return rc;
    }
    return ST_OK;
}

extern "C" int st_predictor_mask(const void *x, int64_t B, int64_t H, const void *A, int64_t r, const void *Bm,
                                 int64_t I, int dtype, float thr, int cmp_ge, float *t_ws, float *scores,
                                 uint8_t *mask, void *stream)
{
    return st_predictor_mask_ex(x, B, H, A, r, Bm, I, dtype, thr, cmp_ge, 0, t_ws, scores, mask, stream);
}
