// Sparse MLP forward in double precision (st_mlp_forward with ST_F64).
//
//   out[b,:] = sum_i act(<x_b, Wg_i>) * <x_b, Wu_i> * Wd_i        i over the n active rows
//
// The reference's operator is dtype-generic on the CPU (torch::matmul, sparse_mlp_op.cpp:151-161) and
// instantiates its CUDA kernels for double as well (sparse_mlp_cuda.cu:90-151); this is the same
// arithmetic for callers that check a model in fp64.  Three plain kernels, every sum in double and in a fixed
// order (results do not depend on the launch):
//   hidden   one wave per active row: the two dot products for up to eight rows of x, activation, product
//   down     a thread per output column and K split: partial[s][b][j] over the split's rows
//   reduce   out[b][j] = partial[0][b][j] + partial[1][b][j] + ...
// FP64 runs on the vector ALUs at a fraction of the rate of the 16-bit paths: this is for checking, not
// serving.
#include "st_common.h"
#include "st_mfma.h"

namespace st {

constexpr int kF64Rows = 8;       // rows of x per pass
constexpr int kF64MaxSplit = 32;  // K splits of the down projection
constexpr int kF64Threads = 256;

__device__ __forceinline__ double activate_f64(double v, int act)
{
    switch (act) {
    case ST_ACT_RELU: return v > 0.0 ? v : 0.0;
    case ST_ACT_SILU: return v / (1.0 + exp(-v));
    case ST_ACT_GELU_TANH: {
        const double k = 0.7978845608028654;  // sqrt(2/pi)
        return 0.5 * v * (1.0 + tanh(k * (v + 0.044715 * v * v * v)));
    }
    case ST_ACT_SIGMOID: return 1.0 / (1.0 + exp(-v));
    default: return v;
    }
}

__device__ __forceinline__ double wave_sum_f64(double v)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    return v;
}

// h[b][i] for the rows b0 .. b0 + nb - 1 of x; one wave per active row i.
template <bool HG>
__global__ __launch_bounds__(kF64Threads) void f64_hidden_kernel(const double *__restrict__ x, int b0, int nb, int H,
                                                                 const double *__restrict__ gate,
                                                                 const double *__restrict__ up, int n_host,
                                                                 const int *__restrict__ n_dev,
                                                                 double *__restrict__ hbuf, long ldh,
                                                                 double *__restrict__ comb, long ldc, int act)
{
    const int n = device_count(n_host, n_dev);
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int i = blockIdx.x * (kF64Threads / kWave) + wave;
    if (i >= n) return;   // (uniform over the wave; no block barrier below)
    double ag[kF64Rows], au[kF64Rows];
#pragma unroll
    for (int b = 0; b < kF64Rows; ++b) ag[b] = au[b] = 0.0;
    const double2 *wg = reinterpret_cast<const double2 *>(HG ? gate + (size_t)i * H : up);
    const double2 *wu = reinterpret_cast<const double2 *>(up + (size_t)i * H);
    const int pairs = H >> 1;
    for (int c = lane; c < pairs; c += kWave) {
        const double2 u = wu[c];
        const double2 g = HG ? wg[c] : u;
#pragma unroll
        for (int b = 0; b < kF64Rows; ++b) {
            if (b < nb) {   // uniform
                const double2 xv = reinterpret_cast<const double2 *>(x + (size_t)(b0 + b) * H)[c];
                au[b] = fma(u.x, xv.x, au[b]);
                au[b] = fma(u.y, xv.y, au[b]);
                if (HG) {
                    ag[b] = fma(g.x, xv.x, ag[b]);
                    ag[b] = fma(g.y, xv.y, ag[b]);
                }
            }
        }
    }
#pragma unroll
    for (int b = 0; b < kF64Rows; ++b) {
        if (b < nb) {
            const double su = wave_sum_f64(au[b]);
            const double sg = HG ? wave_sum_f64(ag[b]) : 0.0;
            if (lane == 0) {
                const double hv = HG ? activate_f64(sg, act) * su : activate_f64(su, act);
                hbuf[(size_t)b * ldh + i] = hv;
                if (comb) {
                    comb[(size_t)(b0 + b) * ldc + i] = hv;
                    if (HG) comb[(size_t)(b0 + b) * ldc + n + i] = su;
                }
            }
        }
    }
}

// partial[s][b][j] = sum over the split's rows i (ascending) of h[b][i] * Wd[i][j]
__global__ __launch_bounds__(kF64Threads) void f64_down_kernel(const double *__restrict__ hbuf, long ldh, int nb, int H,
                                                               const double *__restrict__ down, int n_host,
                                                               const int *__restrict__ n_dev, int split,
                                                               double *__restrict__ partial)
{
    __shared__ double hs[kF64Rows][kF64Threads];
    const int n = device_count(n_host, n_dev);
    const int j = blockIdx.x * kF64Threads + threadIdx.x, s = blockIdx.y;
    const int per = (n + split - 1) / split;
    const int i0 = s * per, i1 = i0 + per < n ? i0 + per : n;
    double acc[kF64Rows];
#pragma unroll
    for (int b = 0; b < kF64Rows; ++b) acc[b] = 0.0;
    for (int t0 = i0; t0 < i1; t0 += kF64Threads) {   // (uniform trip count over the block)
        const int cnt = i1 - t0 < kF64Threads ? i1 - t0 : kF64Threads;
        __syncthreads();
#pragma unroll
        for (int b = 0; b < kF64Rows; ++b)
            if (b < nb && (int)threadIdx.x < cnt) hs[b][threadIdx.x] = hbuf[(size_t)b * ldh + t0 + threadIdx.x];
        __syncthreads();
        if (j < H) {
            for (int t = 0; t < cnt; ++t) {
                const double w = down[(size_t)(t0 + t) * H + j];
#pragma unroll
                for (int b = 0; b < kF64Rows; ++b)
                    if (b < nb) acc[b] = fma(hs[b][t], w, acc[b]);
            }
        }
    }
    if (j < H) {
#pragma unroll
        for (int b = 0; b < kF64Rows; ++b)
            if (b < nb) partial[((size_t)s * kF64Rows + b) * H + j] = acc[b];
    }
}

__global__ __launch_bounds__(kF64Threads) void f64_reduce_kernel(const double *__restrict__ partial, int split, int nb,
                                                                 int H, double *__restrict__ out)
{
    const int j = blockIdx.x * kF64Threads + threadIdx.x, b = blockIdx.y;
    if (j >= H || b >= nb) return;
    double s = partial[(size_t)b * H + j];
    for (int z = 1; z < split; ++z) s += partial[((size_t)z * kF64Rows + b) * H + j];
    out[(size_t)b * H + j] = s;
}

static int f64_split(int H, int n)
{
    const int tiles = (H + kF64Threads - 1) / kF64Threads;
    int s = (2 * device_cu_count() + tiles - 1) / tiles;
    if (s > kF64MaxSplit) s = kF64MaxSplit;
    if (s > (n + 63) / 64) s = (n + 63) / 64;   // at least 64 rows per split
    return s < 1 ? 1 : s;
}

int64_t f64_workspace_bytes(int64_t B, int64_t H, int64_t n)
{
    const int64_t rows = B < kF64Rows ? B : kF64Rows;
    return (rows * n + (int64_t)kF64MaxSplit * kF64Rows * H) * 8;
}

int launch_f64(const void *x, int B, int H, const void *gate, const void *up, const void *down, int n, const int *n_dev,
               void *out, void *comb, long ldc, void *workspace, int act, int has_gate, hipStream_t stream)
{
    const double *xd = static_cast<const double *>(x);
    double *partial = static_cast<double *>(workspace);
    double *hbuf = partial + (size_t)kF64MaxSplit * kF64Rows * H;
    const long ldh = n;
    const int split = f64_split(H, n);
    const int tiles = (H + kF64Threads - 1) / kF64Threads;
    for (int b0 = 0; b0 < B; b0 += kF64Rows) {
        const int nb = B - b0 < kF64Rows ? B - b0 : kF64Rows;
        if (n > 0) {
            ProfScope ps(ST_K_MLP_DECODE, stream);
            const dim3 grid((unsigned)((n + 3) / 4)), block(kF64Threads);
            if (has_gate)
                ST_LAUNCH(ps, f64_hidden_kernel<true>, grid, block, 0, stream, xd, b0, nb, H,
                          static_cast<const double *>(gate), static_cast<const double *>(up), n, n_dev, hbuf, ldh,
                          static_cast<double *>(comb), ldc, act);
            else
                ST_LAUNCH(ps, f64_hidden_kernel<false>, grid, block, 0, stream, xd, b0, nb, H,
                          static_cast<const double *>(nullptr), static_cast<const double *>(up), n, n_dev, hbuf, ldh,
                          static_cast<double *>(comb), ldc, act);
            ST_HIP(hipGetLastError());
        }
        {
            ProfScope ps(ST_K_MLP_DECODE, stream);
            ST_LAUNCH(ps, f64_down_kernel, dim3((unsigned)tiles, (unsigned)split), dim3(kF64Threads), 0, stream, hbuf,
                      ldh, nb, H, static_cast<const double *>(down), n, n_dev, split, partial);
            ST_HIP(hipGetLastError());
        }
        {
            ProfScope ps(ST_K_MLP_REDUCE, stream);
            ST_LAUNCH(ps, f64_reduce_kernel, dim3((unsigned)tiles, (unsigned)nb), dim3(kF64Threads), 0, stream, partial,
                      split, nb, H, static_cast<double *>(out) + (size_t)b0 * H);
            ST_HIP(hipGetLastError());
        }
    }
    return ST_OK;
}

}  // namespace st

extern "C" int64_t st_mlp_f64_workspace_bytes(int64_t B, int64_t H, int64_t n)
{
    if (B < 1 || H < 1 || n < 0) return 0;
    return st::f64_workspace_bytes(B, H, n);
}
