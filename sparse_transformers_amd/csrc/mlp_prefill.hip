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
// of up), 4 waves of 64 x 64, K stage 128 (four MFMA steps), one LDS stage with
// the next stage's global loads held in registers during the MFMAs.
//
// The reference only runs the sparse path for decode (src/modeling_skip.py:236);
// this is the same contraction as sparse_mlp_forward_cpu
// (sparse_transformers/csrc/sparse_mlp_op.cpp:151-161) for B > 1 rows.
#include "st_mfma.h"

namespace st {

constexpr int kPfThreads = 256;
constexpr int kPfBM = 128;   // rows of x per block
constexpr int kPfBN = 128;   // output columns per block (kernel 1: 64 gate + 64 up rows)
constexpr int kPfBK = 128;   // K per stage = 4 MFMA steps; 256 contiguous bytes per row and stage
constexpr int kPfKB = kPfBK / 32;
constexpr int kPfCh = kPfBK / 8;   // 16-byte chunks per row and stage
constexpr int kPfLd = kPfCh + 1;   // LDS row stride in 16-byte units (one pad chunk spreads the banks)

constexpr int kXcds = 8;

// Workgroups are handed to the 8 XCDs round-robin by their linear id, and each XCD has its own L2.
// This maps the linear id to a tile id such that every XCD works through one contiguous range of tile
// ids; tile ids are ordered so that neighbours share an operand tile (the same weight rows for all row
// tiles of x), which then comes from that XCD's L2 instead of HBM.  Returns -1 for the padding ids.
__device__ __forceinline__ int xcd_tile_id(int bid, int ntiles)
{
    const int per = (ntiles + kXcds - 1) / kXcds;
    const int t = (bid % kXcds) * per + bid / kXcds;
    return (bid / kXcds < per && t < ntiles) ? t : -1;
}

// Each stage moves 256 contiguous bytes of every row from HBM/L2 into LDS (a short K step would pay a
// full memory latency for 64 bytes per row); the next stage's loads are in flight during the MFMAs.

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
                                                                    int has_gate, int jt, int mt)
{
    __shared__ uint4 sX[kPfBM][kPfLd];
    __shared__ uint4 sG[64][kPfLd];
    __shared__ uint4 sU[64][kPfLd];

    const int n = device_count(n_host, n_dev);
    const int n_pad = (n + kPfBK - 1) / kPfBK * kPfBK;  // kernel 2 runs whole K stages over Hh
    const int tile = xcd_tile_id(blockIdx.x, jt * mt);   // row tiles of x fastest: they share the weight rows
    if (tile < 0) return;
    const int j0 = (tile / mt) * 64, m0 = (tile % mt) * kPfBM;
    if (j0 >= n_pad) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // global -> register staging: thread owns chunk `ch` of rows r0 + 16 i
    const int ch = tid & (kPfCh - 1), r0 = tid / kPfCh;
    constexpr int kRowStep = kPfThreads / kPfCh;   // 16
    constexpr int kXL = kPfBM / kRowStep;          // 8 loads for x
    constexpr int kWL = 64 / kRowStep;             // 4 loads for gate, 4 for up

    f32x4_t ag[4][2], au[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ag[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            au[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }

    // Loads are unconditional (rows clamped into range): rows of x beyond M only feed outputs that are
    // never stored, weight rows beyond n only feed columns that are written as zeros below.
    int xoff[kXL], woff[kWL];
#pragma unroll
    for (int i = 0; i < kXL; ++i) {
        const int r = m0 + r0 + kRowStep * i;
        xoff[i] = (r < M ? r : M - 1) * H + ch * 8;
    }
#pragma unroll
    for (int i = 0; i < kWL; ++i) {
        const int r = j0 + r0 + kRowStep * i;
        woff[i] = (r < n ? r : (n > 0 ? n - 1 : 0)) * H + ch * 8;
    }
    uint4 rx[kXL], rg[kWL], ru[kWL];
    auto gload = [&](int k0) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kXL; ++i) rx[i] = ld16(X + xoff[i] + k0);
#pragma unroll
        for (int i = 0; i < kWL; ++i) {
            ru[i] = ld16(up + woff[i] + k0);
            rg[i] = has_gate ? ld16(gate + woff[i] + k0) : zero4;
        }
    };
    auto sstore = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kXL; ++i) sX[r0 + kRowStep * i][ch] = rx[i];
#pragma unroll
        for (int i = 0; i < kWL; ++i) {
            sG[r0 + kRowStep * i][ch] = rg[i];
            sU[r0 + kRowStep * i][ch] = ru[i];
        }
    };

    const int nk = (H + kPfBK - 1) / kPfBK;
    gload(0);
    for (int ks = 0; ks < nk; ++ks) {
        sstore();
        __syncthreads();
        if (ks + 1 < nk) gload((ks + 1) * kPfBK);
#pragma unroll
        for (int kb = 0; kb < kPfKB; ++kb) {
            uint4 fa[4], fg[2], fu[2];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = sX[64 * wm + 16 * i + l16][4 * kb + q];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                fg[j] = sG[32 * wn + 16 * j + l16][4 * kb + q];
                fu[j] = sU[32 * wn + 16 * j + l16][4 * kb + q];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    au[i][j] = Mfma<T>::run(fa[i], fu[j], au[i][j]);
                    if (has_gate) ag[i][j] = Mfma<T>::run(fa[i], fg[j], ag[i][j]);
                }
        }
        __syncthreads();
    }

    // D[m][j]: lane holds rows 4*q + e (e = 0..3) of column l16 in every 16 x 16 block.
    // Columns n .. n_pad are written as zeros so that kernel 2 can run whole K stages.
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
                                                                  int split_k, int ct, int mt)
{
    __shared__ uint4 sA[kPfBM][kPfLd];
    __shared__ uint32_t sB[kPfBN][kPfLd * 4];  // [column][k pairs]: Wd^T tile

    const int n = device_count(n_host, n_dev);
    const int tile = xcd_tile_id(blockIdx.x, ct * mt * split_k);  // row tiles fastest, then column tiles, then splits
    if (tile < 0) return;
    const int z = tile / (ct * mt), c0 = ((tile / mt) % ct) * kPfBN, m0 = (tile % mt) * kPfBM;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // K range of this split, in whole K stages
    const int nk_all = (n + kPfBK - 1) / kPfBK;
    const int per = (nk_all + split_k - 1) / split_k;
    const int ks0 = z * per, ks1 = (ks0 + per < nk_all) ? ks0 + per : nk_all;

    const int ch = tid & (kPfCh - 1), r0 = tid / kPfCh;
    constexpr int kRowStep = kPfThreads / kPfCh;   // 16
    constexpr int kAL = kPfBM / kRowStep;          // 8 loads for Hh
    // Wd tile: this thread owns the row pairs kp + 16 i (rows 2 kp', 2 kp' + 1) and 8 columns
    const int kp = tid & 15, cg = tid >> 4;
    constexpr int kBP = kPfBK / 2 / 16;            // 4 row pairs per thread
    const bool cok = c0 + 8 * cg < H;

    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Unconditional loads from clamped rows; rows of Wd at or beyond n are replaced by zeros (they meet
    // the zero padding of Hh, but stale rows may hold anything, and 0 * inf is not 0).
    int aoff[kAL];
#pragma unroll
    for (int i = 0; i < kAL; ++i) {
        const int r = m0 + r0 + kRowStep * i;
        aoff[i] = (int)((r < M ? r : M - 1) * ldh) + ch * 8;
    }
    const int ccol = cok ? c0 + 8 * cg : 0;
    const int nlast = n > 0 ? n - 1 : 0;
    uint4 ra[kAL], rb[kBP][2];
    auto gload = [&](int ks) __attribute__((always_inline)) {
        const int k0 = ks * kPfBK;
#pragma unroll
        for (int i = 0; i < kAL; ++i) ra[i] = ld16(Hh + aoff[i] + k0);
#pragma unroll
        for (int i = 0; i < kBP; ++i) {
            const int r = k0 + 2 * (kp + 16 * i);
            const int ra0 = r < n ? r : nlast, ra1 = r + 1 < n ? r + 1 : nlast;
            rb[i][0] = ld16(Wd + (size_t)ra0 * H + ccol);
            rb[i][1] = ld16(Wd + (size_t)ra1 * H + ccol);
            if (!(cok && r < n)) rb[i][0] = zero4;
            if (!(cok && r + 1 < n)) rb[i][1] = zero4;
        }
    };
    auto sstore = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kAL; ++i) sA[r0 + kRowStep * i][ch] = ra[i];
#pragma unroll
        for (int i = 0; i < kBP; ++i) {
            const uint32_t lo[4] = {rb[i][0].x, rb[i][0].y, rb[i][0].z, rb[i][0].w};
            const uint32_t hi[4] = {rb[i][1].x, rb[i][1].y, rb[i][1].z, rb[i][1].w};
#pragma unroll
            for (int v = 0; v < 4; ++v) {  // word v holds columns 2v, 2v+1 of one row
                sB[8 * cg + 2 * v][kp + 16 * i] = (lo[v] & 0xffffu) | (hi[v] << 16);
                sB[8 * cg + 2 * v + 1][kp + 16 * i] = (lo[v] >> 16) | (hi[v] & 0xffff0000u);
            }
        }
    };

    if (ks0 < ks1) gload(ks0);
    for (int ks = ks0; ks < ks1; ++ks) {
        sstore();
        __syncthreads();
        if (ks + 1 < ks1) gload(ks + 1);
#pragma unroll
        for (int kb = 0; kb < kPfKB; ++kb) {
            uint4 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = sA[64 * wm + 16 * i + l16][4 * kb + q];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                fb[j] = *reinterpret_cast<const uint4 *>(&sB[64 * wn + 16 * j + l16][16 * kb + 4 * q]);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
        }
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
    if (s > nk / 4) s = nk / 4;  // keep at least 4 K stages per split
    if (s < 1) s = 1;
    if (s > 16) s = 16;
    return s;
}

int64_t prefill_ldh(int64_t n) { return (n + kPfBK - 1) / kPfBK * kPfBK; }

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
        const int jt = (int)(ldh / 64), mt = (M + kPfBM - 1) / kPfBM;
        const int grid = (jt * mt + kXcds - 1) / kXcds * kXcds;
        ST_LAUNCH(ps, prefill_gateup_kernel<T>, dim3(grid), dim3(kPfThreads), 0, stream,
                           static_cast<const T *>(x), M, H, static_cast<const T *>(gate), static_cast<const T *>(up), n,
                           n_dev, Hh, ldh, static_cast<T *>(comb), ldc, act, has_gate, jt, mt);
    }
    ST_HIP(hipGetLastError());
    {
        ProfScope ps(ST_K_MLP_PREFILL_DOWN, stream);
        const int ct = (H + kPfBN - 1) / kPfBN, mt = (M + kPfBM - 1) / kPfBM;
        const int grid = (ct * mt * split_k + kXcds - 1) / kXcds * kXcds;
        ST_LAUNCH(ps, prefill_down_kernel<T>, dim3(grid), dim3(kPfThreads), 0, stream, Hh, ldh, M,
                           static_cast<const T *>(down), H, n, n_dev, static_cast<T *>(out), partial, split_k, ct, mt);
    }
    ST_HIP(hipGetLastError());
    if (split_k > 1) {
        ProfScope ps(ST_K_MLP_REDUCE, stream);
        const size_t quads = ((size_t)M * H + 3) / 4;
        ST_LAUNCH(ps, prefill_reduce_kernel<T>, dim3((unsigned)((quads + 255) / 256)), dim3(256), 0, stream,
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
