// Sparse MLP over the active set for many rows of x (prefill / large batch):
// a dense contraction, so it runs on the matrix cores (fp16 / bf16 MFMA
// 16x16x32, fp32 accumulate).
//
//   kernel 1  Hh[M,n] = act(X Wg^T) * (X Wu^T)       X [M,H], Wg/Wu [n,H]
//             both operands are K-contiguous, tiles go global -> LDS as is;
//             gate and up share the X fragments, the activation is applied
//             to the accumulators before Hh is written
//   kernel 2  Out[M,H] = Hh[M,n] Wd[n,H]              Wd rows are the packed
//             down columns, i.e. K runs down the rows: pairs of rows are
//             interleaved in registers so that LDS holds Wd^T tiles
//             ([column][k]) and the fragment reads stay 16-byte
// Block tile 128 x 128 (kernel 1: 128 rows of x by 64 active rows of gate and
// of up), 4 waves of 64 x 64, K step 32, LDS double-buffered with the next
// step's global loads in flight during the MFMAs.
//
// The reference only runs the sparse path for decode (src/modeling_skip.py:236);
// this is the same contraction as sparse_mlp_forward_cpu
// (sparse_transformers/csrc/sparse_mlp_op.cpp:151-161) for B > 1 rows.
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

constexpr int kPfThreads = 256;
constexpr int kPfBM = 128;  // rows of x per block
constexpr int kPfBN = 128;  // output columns per block (kernel 1: 64 gate + 64 up rows)
constexpr int kPfBK = 32;   // K step = one MFMA
constexpr int kPfLd = 5;    // LDS row stride in 16-byte units: 4 used + 1 pad (bank spread)

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

// ---------------------------------------------------------------------------
// kernel 1: gate / up projections + activation
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kPfThreads) void prefill_gateup_kernel(const T *__restrict__ X, int M, int H,
                                                                    const T *__restrict__ gate,
                                                                    const T *__restrict__ up, int n_host,
                                                                    const int *__restrict__ n_dev,
                                                                    T *__restrict__ Hh, long ldh,
                                                                    T *__restrict__ comb, long ldc, int act,
                                                                    int has_gate)
{
    __shared__ uint4 sX[2][kPfBM][kPfLd];
    __shared__ uint4 sG[2][64][kPfLd];
    __shared__ uint4 sU[2][64][kPfLd];

    const int n = device_count(n_host, n_dev);
    const int j0 = blockIdx.x * 64, m0 = blockIdx.y * kPfBM;
    if (j0 >= n) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // global -> register staging: X 2 chunks per thread, gate / up 1 chunk each
    const int xr0 = tid >> 2, xr1 = (tid + kPfThreads) >> 2, ch = tid & 3;
    const bool xok0 = m0 + xr0 < M, xok1 = m0 + xr1 < M, wok = j0 + xr0 < n;
    const T *xp0 = X + (size_t)(m0 + xr0) * H + ch * 8;
    const T *xp1 = X + (size_t)(m0 + xr1) * H + ch * 8;
    const T *gp = gate + (size_t)(j0 + xr0) * H + ch * 8;
    const T *upp = up + (size_t)(j0 + xr0) * H + ch * 8;

    f32x4_t ag[4][2], au[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ag[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            au[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }

    uint4 rx0, rx1, rg, ru;
    auto gload = [&](int k0) {
        rx0 = xok0 ? ld16(xp0 + k0) : zero4;
        rx1 = xok1 ? ld16(xp1 + k0) : zero4;
        ru = wok ? ld16(upp + k0) : zero4;
        rg = (wok && has_gate) ? ld16(gp + k0) : zero4;
    };
    auto sstore = [&](int buf) {
        sX[buf][xr0][ch] = rx0;
        sX[buf][xr1][ch] = rx1;
        sG[buf][xr0][ch] = rg;
        sU[buf][xr0][ch] = ru;
    };

    const int nk = H / kPfBK;
    gload(0);
    sstore(0);
    __syncthreads();
    for (int ks = 0; ks < nk; ++ks) {
        const int buf = ks & 1;
        if (ks + 1 < nk) gload((ks + 1) * kPfBK);
        uint4 fa[4], fg[2], fu[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = sX[buf][64 * wm + 16 * i + l16][q];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            fg[j] = sG[buf][32 * wn + 16 * j + l16][q];
            fu[j] = sU[buf][32 * wn + 16 * j + l16][q];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                au[i][j] = Mfma<T>::run(fa[i], fu[j], au[i][j]);
                if (has_gate) ag[i][j] = Mfma<T>::run(fa[i], fg[j], ag[i][j]);
            }
        if (ks + 1 < nk) sstore(buf ^ 1);
        __syncthreads();
    }

    // D[m][j]: lane holds rows 4*q + e (e = 0..3) of column l16 in every 16 x 16 block.
    // Columns n .. round_up(n, 32) are written as zeros so that kernel 2 can run whole K steps.
    const int n_pad = (n + kPfBK - 1) / kPfBK * kPfBK;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int col = j0 + 32 * wn + 16 * j + l16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + 64 * wm + 16 * i + 4 * q + e;
                if (m < M && col < n_pad) {
                    float hv = 0.f;
                    if (col < n) hv = has_gate ? activate(ag[i][j][e], act) * au[i][j][e] : activate(au[i][j][e], act);
                    Hh[(size_t)m * ldh + col] = from_float<T>(hv);
                    if (comb && col < n) comb[(size_t)m * ldc + col] = from_float<T>(hv);
                }
            }
        }
}

// ---------------------------------------------------------------------------
// kernel 2: down projection
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kPfThreads) void prefill_down_kernel(const T *__restrict__ Hh, long ldh, int M,
                                                                  const T *__restrict__ Wd, int H, int n_host,
                                                                  const int *__restrict__ n_dev,
                                                                  T *__restrict__ Out, float *__restrict__ partial,
                                                                  int split_k)
{
    __shared__ uint4 sA[2][kPfBM][kPfLd];
    __shared__ uint32_t sB[2][kPfBN][kPfLd * 4];  // [column][k pairs]: Wd^T tile

    const int n = device_count(n_host, n_dev);
    const int c0 = blockIdx.x * kPfBN, m0 = blockIdx.y * kPfBM, z = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // K range of this split, in whole K steps
    const int nk_all = (n + kPfBK - 1) / kPfBK;
    const int per = (nk_all + split_k - 1) / split_k;
    const int ks0 = z * per, ks1 = (ks0 + per < nk_all) ? ks0 + per : nk_all;

    const int ar0 = tid >> 2, ar1 = (tid + kPfThreads) >> 2, ch = tid & 3;
    const bool aok0 = m0 + ar0 < M, aok1 = m0 + ar1 < M;
    const T *ap0 = Hh + (size_t)(m0 + ar0) * ldh + ch * 8;
    const T *ap1 = Hh + (size_t)(m0 + ar1) * ldh + ch * 8;
    // Wd tile: this thread owns the row pair (2 kp, 2 kp + 1) and 8 columns
    const int kp = tid & 15, cg = tid >> 4;
    const bool cok = c0 + 8 * cg < H;
    const T *bp = Wd + (size_t)(2 * kp) * H + c0 + 8 * cg;

    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    uint4 ra0, ra1, rb0, rb1;
    auto gload = [&](int ks) {
        const int k0 = ks * kPfBK;
        ra0 = aok0 ? ld16(ap0 + k0) : zero4;
        ra1 = aok1 ? ld16(ap1 + k0) : zero4;
        const int r = k0 + 2 * kp;
        rb0 = (cok && r < n) ? ld16(bp + (size_t)k0 * H) : zero4;
        rb1 = (cok && r + 1 < n) ? ld16(bp + (size_t)(k0 + 1) * H) : zero4;
    };
    auto sstore = [&](int buf) {
        sA[buf][ar0][ch] = ra0;
        sA[buf][ar1][ch] = ra1;
        const uint32_t lo[4] = {rb0.x, rb0.y, rb0.z, rb0.w}, hi[4] = {rb1.x, rb1.y, rb1.z, rb1.w};
#pragma unroll
        for (int v = 0; v < 4; ++v) {  // word v holds columns 2v, 2v+1 of one row
            sB[buf][8 * cg + 2 * v][kp] = (lo[v] & 0xffffu) | (hi[v] << 16);
            sB[buf][8 * cg + 2 * v + 1][kp] = (lo[v] >> 16) | (hi[v] & 0xffff0000u);
        }
    };

    if (ks0 < ks1) {
        gload(ks0);
        sstore(0);
    }
    __syncthreads();
    for (int ks = ks0; ks < ks1; ++ks) {
        const int buf = (ks - ks0) & 1;
        if (ks + 1 < ks1) gload(ks + 1);
        uint4 fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = sA[buf][64 * wm + 16 * i + l16][q];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            fb[j] = *reinterpret_cast<const uint4 *>(&sB[buf][64 * wn + 16 * j + l16][4 * q]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
        if (ks + 1 < ks1) sstore(buf ^ 1);
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = c0 + 64 * wn + 16 * j + l16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int m = m0 + 64 * wm + 16 * i + 4 * q + e;
                if (m < M && col < H) {
                    if (split_k == 1) Out[(size_t)m * H + col] = from_float<T>(acc[i][j][e]);
                    else partial[((size_t)z * M + m) * H + col] = acc[i][j][e];
                }
            }
        }
}

// out[m, c] = sum over splits of partial[z][m][c]
template <typename T>
__global__ __launch_bounds__(256) void prefill_reduce_kernel(const float *__restrict__ partial, int split_k, int M,
                                                             int H, T *__restrict__ out)
{
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4, total = (size_t)M * H;
    if (i4 >= total) return;
    float4 s = *reinterpret_cast<const float4 *>(partial + i4);
    for (int z = 1; z < split_k; ++z) {
        const float4 v = *reinterpret_cast<const float4 *>(partial + (size_t)z * total + i4);
        s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
    }
    T *o = out + i4;
    o[0] = from_float<T>(s.x); o[1] = from_float<T>(s.y); o[2] = from_float<T>(s.z); o[3] = from_float<T>(s.w);
}

int prefill_split_k(int M, int H, int n)
{
    const int tiles = ((M + kPfBM - 1) / kPfBM) * ((H + kPfBN - 1) / kPfBN);
    int s = (2 * device_cu_count() + tiles - 1) / tiles;  // aim at two blocks per CU
    const int nk = (n + kPfBK - 1) / kPfBK;
    if (s > nk / 8) s = nk / 8;  // keep at least 8 K steps per split
    if (s < 1) s = 1;
    if (s > 16) s = 16;
    return s;
}

int64_t prefill_ldh(int64_t n) { return (n + 63) / 64 * 64; }

int64_t prefill_workspace_bytes(int64_t M, int64_t H, int64_t n)
{
    const int64_t hh = M * prefill_ldh(n) * 2;
    const int64_t part = (int64_t)16 * M * H * 4;  // upper bound on the split count
    return ((hh + 255) & ~(int64_t)255) + part;
}

template <typename T>
static int launch_prefill_t(const void *x, int M, int H, const void *gate, const void *up, const void *down, int n,
                            const int *n_dev, void *out, void *comb, long ldc, void *workspace, int act, int has_gate,
                            hipStream_t stream)
{
    const long ldh = (long)prefill_ldh(n);
    T *Hh = static_cast<T *>(workspace);
    const int64_t hh_bytes = (((int64_t)M * ldh * 2) + 255) & ~(int64_t)255;
    float *partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + hh_bytes);
    const int split_k = prefill_split_k(M, H, n);
    {
        ProfScope ps(ST_K_MLP_PREFILL_GATEUP, stream);
        hipLaunchKernelGGL(prefill_gateup_kernel<T>, dim3((n + 63) / 64, (M + kPfBM - 1) / kPfBM), dim3(kPfThreads),
                           0, stream, static_cast<const T *>(x), M, H, static_cast<const T *>(gate),
                           static_cast<const T *>(up), n, n_dev, Hh, ldh, static_cast<T *>(comb), ldc, act, has_gate);
    }
    ST_HIP(hipGetLastError());
    {
        ProfScope ps(ST_K_MLP_PREFILL_DOWN, stream);
        hipLaunchKernelGGL(prefill_down_kernel<T>, dim3((H + kPfBN - 1) / kPfBN, (M + kPfBM - 1) / kPfBM, split_k),
                           dim3(kPfThreads), 0, stream, Hh, ldh, M, static_cast<const T *>(down), H, n, n_dev,
                           static_cast<T *>(out), partial, split_k);
    }
    ST_HIP(hipGetLastError());
    if (split_k > 1) {
        ProfScope ps(ST_K_MLP_REDUCE, stream);
        const size_t quads = ((size_t)M * H + 3) / 4;
        hipLaunchKernelGGL(prefill_reduce_kernel<T>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream,
                           partial, split_k, M, H, static_cast<T *>(out));
        ST_HIP(hipGetLastError());
    }
    return ST_OK;
}

int launch_prefill(int dtype, const void *x, int M, int H, const void *gate, const void *up, const void *down, int n,
                   const int *n_dev, void *out, void *comb, long ldc, void *workspace, int act, int has_gate,
                   hipStream_t stream)
{
    if (dtype == ST_F16)
        return launch_prefill_t<f16_t>(x, M, H, gate, up, down, n, n_dev, out, comb, ldc, workspace, act, has_gate,
                                       stream);
    return launch_prefill_t<bf16_t>(x, M, H, gate, up, down, n, n_dev, out, comb, ldc, workspace, act, has_gate,
                                    stream);
}

}  // namespace st
