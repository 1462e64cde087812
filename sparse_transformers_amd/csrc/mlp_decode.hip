// Fused sparse-MLP decode kernel for gfx950 (small batch, HBM-bound).
//
// One launch streams the three packed active matrices exactly once.  A block
// (one per CU) owns the active rows j with j % gridDim.x == blockIdx.x.  Every
// thread owns one 16-byte column chunk of the hidden dimension (two for very
// wide rows) and, for each row its thread group has in flight, issues the
// gate, up AND down loads of that chunk together.  Rows are processed in
// batches of RB per group through two register buffers: while one batch is
// being computed the loads of the next are in flight, so the memory system is
// kept busy through the reductions and barriers of the previous batch.
//   phase 1  per-thread partial products <gate[j],x>, <up[j],x> on the chunk,
//            DPP wave reduction, cross-wave sum through LDS,
//            h[j] = act(g) * u  left in LDS
//   phase 2  acc[chunk] += h[j] * down[j, chunk]   from the registers that
//            were loaded before phase 1
// Each block writes one fp32 partial row; a second small kernel sums the
// partials in a fixed order (deterministic) and converts to the output type.
//
// Replaces sparse_mlp_forward_cpu (sparse_transformers/csrc/sparse_mlp_op.cpp:79-192)
// and SkipMLP._forward_sparse_weight_cache (src/modeling_skip.py:114-117).
#include "st_common.h"

#include <atomic>

#include <cstdlib>
#include <mutex>

namespace st {

// Scratch of the entry point that allocates nothing (st_mlp_forward_static): the fp32 partial rows
// [blocks][rows of x][H] of the streaming decode kernel.  One copy per GPU the library runs on, held until
// the process ends.  In host code this name is only a handle for hipGetSymbolAddress; kernels get the
// address that call returns.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

template <int RB, int CPT> struct RowBatch {
    uint4 g[RB][CPT], u[RB][CPT], d[RB][CPT];
};

// T: storage type; NB: x rows per launch; RB: rows per group in one register
// buffer; CPT: 16-byte chunks per thread; TPB: threads per block (512 leaves
// 256 VGPRs per thread, 1024 leaves 128); DB: two register buffers (the next
// batch is in flight while one is computed) or one (a single deep batch, which
// measures faster when all rows of a block fit in it).
template <typename T, int NB, int RB, int CPT, int TPB, bool DB>
__global__ __launch_bounds__(TPB) void mlp_decode_kernel(
    const T *__restrict__ x, const T *__restrict__ gate, const T *__restrict__ up, const T *__restrict__ down,
    const int *__restrict__ n_dev, int H, int launch_word, int n_spec, int n_host, T *__restrict__ combined,
    long ldc, float *__restrict__ partials, int act)
{
    // (the first 14 dwords of the arguments are in scalar registers when the wave starts: everything the first loads
    // need is among them -- the number of blocks, the thread-group size, the gate flag and the rows of x share one
    // dword, and the host passes the row count to request ahead of the device's count, `n_spec`, ready-made; later
    // arguments arrive by a load)
    const int G = launch_word & 0xffff, gs_log2 = (launch_word >> 16) & 15, B = (launch_word >> 24) & 15;
    const bool has_gate = ((launch_word >> 20) & 1) != 0;
    constexpr int VEC = Elem<T>::kVec;
    extern __shared__ __align__(16) unsigned char region[];  // group combine buffer
    __shared__ float red[TPB / kWave][RB][NB][2];             // per-wave partial (g,u)
    __shared__ float hs[TPB / kWave][RB][NB];                 // h of the rows being computed

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int blk = blockIdx.x;
    // Active count: requested first, consumed only after the first two batches
    // of weight loads have been issued.  Rows are dealt to blocks round-robin,
    // so which rows a block owns does not depend on the count, and rows below
    // `n_spec` can be requested before the count has arrived (the active
    // buffers hold I rows, so this is safe).
    ST_TL(0);
    const int nd_raw = n_dev ? *n_dev : n_host;
    const int chunks = H / VEC;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // groups of 2^gs_log2 threads each cover all chunks of a row
    const int GS = 1 << gs_log2, ngrp = TPB >> gs_log2, wpg = GS >> 6;
    const int grp = tid >> gs_log2, cc = tid & (GS - 1);
    bool valid[CPT];
    size_t coff[CPT];
#pragma unroll
    for (int q = 0; q < CPT; ++q) {
        valid[q] = cc + q * GS < chunks;
        coff[q] = valid[q] ? (size_t)(cc + q * GS) * VEC : 0;   // clamped: loads below are unconditional
    }

    // a wave whose 64 chunks all lie past the row end (H/VEC not a power of two) loads nothing (scalar test)
    const bool wave_live = __builtin_amdgcn_readfirstlane(cc & ~(kWave - 1)) < chunks;

    uint4 xr[NB][CPT];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int q = 0; q < CPT; ++q) {
            xr[b][q] = ld16(x + (size_t)(b < B ? b : 0) * H + coff[q]);
            if (!(valid[q] && b < B)) xr[b][q] = zero4;
        }

    // row of (batch, slot k) for this thread's group
    auto row_of = [&](int bat, int k) { return blk + G * (grp + ngrp * (bat * RB + k)); };
    // Loads are issued unconditionally from a clamped row / chunk: a branch around every load costs far
    // more than a few duplicate (cache-hit) loads.  What a clamped load returns is never used: x is zero
    // on chunks past the row end, h is forced to zero for rows >= n, and the down row is replaced by
    // zeros where it is consumed.  limit >= 1.
    auto load_batch = [&](RowBatch<RB, CPT> &w, int bat, int limit) __attribute__((always_inline)) {
        if (!wave_live) return;
#pragma unroll
        for (int k = 0; k < RB; ++k) {
            const int row = row_of(bat, k);
            const size_t ro = (size_t)(row < limit ? row : limit - 1) * H;
#pragma unroll
            for (int q = 0; q < CPT; ++q) {
                const size_t o = ro + coff[q];
                w.u[k][q] = ld16_stream(up + o);
                w.d[k][q] = ld16_stream(down + o);
                w.g[k][q] = has_gate ? ld16_stream(gate + o) : zero4;
            }
        }
    };
    auto zero_batch = [&](RowBatch<RB, CPT> &w) __attribute__((always_inline)) {
#pragma unroll
        for (int k = 0; k < RB; ++k)
#pragma unroll
            for (int q = 0; q < CPT; ++q) { w.g[k][q] = zero4; w.u[k][q] = zero4; w.d[k][q] = zero4; }
    };

    RowBatch<RB, CPT> w0, w1;
    if (n_spec > 0 && wave_live) {
        load_batch(w0, 0, n_spec);
        if constexpr (DB) load_batch(w1, 1, n_spec);
    } else {
        zero_batch(w0);
        if constexpr (DB) zero_batch(w1);
    }
    ST_TL(1);
    int n = nd_raw < n_host ? nd_raw : n_host;
    if (n < 0) n = 0;

    float acc[NB][CPT][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int q = 0; q < CPT; ++q)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[b][q][e] = 0.f;

    auto compute = [&](const RowBatch<RB, CPT> &w, int bat) {
        // ---- phase 1: partial dot products on this thread's chunk(s)
        float pg[RB][NB], pu[RB][NB];
#pragma unroll
        for (int k = 0; k < RB; ++k) {
#pragma unroll
            for (int b = 0; b < NB; ++b) pg[k][b] = pu[k][b] = 0.f;
#pragma unroll
            for (int q = 0; q < CPT; ++q)
#pragma unroll
                for (int b = 0; b < NB; ++b) dot_chunk<T>(w.g[k][q], w.u[k][q], xr[b][q], pg[k][b], pu[k][b]);
        }
#pragma unroll
        for (int k = 0; k < RB; ++k)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const float sg = wave_sum_dpp(pg[k][b]);
                const float su = wave_sum_dpp(pu[k][b]);
                if (lane == 0) {
                    red[wave][k][b][0] = sg;
                    red[wave][k][b][1] = su;
                }
            }
        ST_TL(2);
        __syncthreads();
        ST_TL(3);
        if (tid < ngrp * RB * NB) {
            const int g_ = tid / (RB * NB), rem = tid - g_ * (RB * NB);
            const int k_ = rem / NB, b_ = rem - k_ * NB;
            const int row = blk + G * (g_ + ngrp * (bat * RB + k_));
            float sg = 0.f, su = 0.f;
            for (int wv = g_ * wpg; wv < (g_ + 1) * wpg; ++wv) {
                sg += red[wv][k_][b_][0];
                su += red[wv][k_][b_][1];
            }
            const float hv = has_gate ? activate(sg, act) * su : activate(su, act);
            const bool ok = row < n;
            hs[g_][k_][b_] = ok ? hv : 0.f;
            if (ok && combined && b_ < B) {
                combined[(size_t)b_ * ldc + row] = from_float<T>(hv);
                if (has_gate) combined[(size_t)b_ * ldc + n + row] = from_float<T>(su);
            }
        }
        __syncthreads();
        ST_TL(4);
        // ---- phase 2: down projection from the rows already in registers
#pragma unroll
        for (int k = 0; k < RB; ++k) {
            const bool row_ok = row_of(bat, k) < n;
#pragma unroll
            for (int q = 0; q < CPT; ++q) {
                const uint4 wsel = row_ok ? w.d[k][q] : zero4;   // rows past the count may hold anything
#pragma unroll
                for (int b = 0; b < NB; ++b) axpy_chunk<T>(hs[grp][k][b], wsel, acc[b][q]);
            }
        }
    };

    const int jcount = n > blk ? (n - blk + G - 1) / G : 0;      // rows of this block
    const int nbat = ((jcount + ngrp - 1) / ngrp + RB - 1) / RB;  // uniform over the block
    if (n != n_spec && nbat > 0) {  // the host's guess was off: request the first batches again with the true count
        load_batch(w0, 0, n);
        if constexpr (DB) load_batch(w1, 1, n);
    }
    if constexpr (DB) {
        for (int bat = 0; bat < nbat; bat += 2) {
            compute(w0, bat);
            if (bat + 2 < nbat) load_batch(w0, bat + 2, n);
            if (bat + 1 < nbat) {
                compute(w1, bat + 1);
                if (bat + 3 < nbat) load_batch(w1, bat + 3, n);
            }
        }
    } else {
        for (int bat = 0; bat < nbat; ++bat) {
            if (bat > 0) load_batch(w0, bat, n);
            compute(w0, bat);
        }
    }

    ST_TL(5);
    // ---- combine the thread groups through LDS (CPT == 1 whenever ngrp > 1)
    if (ngrp > 1) {
        float *redc = reinterpret_cast<float *>(region);  // [ngrp-1][NB][H]
        if (grp > 0 && valid[0]) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < VEC; e += 4)
                    *reinterpret_cast<float4 *>(redc + ((size_t)(grp - 1) * NB + b) * H + coff[0] + e) =
                        make_float4(acc[b][0][e], acc[b][0][e + 1], acc[b][0][e + 2], acc[b][0][e + 3]);
        }
        __syncthreads();
        if (grp == 0 && valid[0]) {
            for (int gq = 1; gq < ngrp; ++gq)
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int e = 0; e < VEC; e += 4) {
                        const float4 v =
                            *reinterpret_cast<const float4 *>(redc + ((size_t)(gq - 1) * NB + b) * H + coff[0] + e);
                        acc[b][0][e] += v.x; acc[b][0][e + 1] += v.y; acc[b][0][e + 2] += v.z; acc[b][0][e + 3] += v.w;
                    }
        }
    }
    if (grp == 0) {
#pragma unroll
        for (int q = 0; q < CPT; ++q) {
            if (!valid[q]) continue;
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < VEC; e += 4)
                    *reinterpret_cast<float4 *>(partials + ((size_t)blk * NB + b) * H + coff[q] + e) =
                        make_float4(acc[b][q][e], acc[b][q][e + 1], acc[b][q][e + 2], acc[b][q][e + 3]);
        }
    }
    ST_TL(6);
}

// out[b, c] = sum over blocks of partials[blk][b][c], fixed order.  CW threads share a row of 4 * CW columns,
// 256 / CW groups of threads take the partial rows round-robin, U rows per thread requested together (one
// memory round trip for G <= 256).
constexpr int kReduceThreads = 128;   // measured against 64 / 256 / 512 threads per block
template <typename T, int CW>
__global__ __launch_bounds__(kReduceThreads) void mlp_reduce_kernel(const float *__restrict__ partials, int G, int NB, int B,
                                                         int H, T *__restrict__ out)
{
    constexpr int RG = kReduceThreads / CW, U = 256 / RG;
    __shared__ float4 red[RG][CW];
    const int tid = threadIdx.x, q = tid % CW, rg = tid / CW;
    const int b = blockIdx.y;
    const int col = blockIdx.x * (4 * CW) + q * 4;
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    if (col < H) {
        for (int blk0 = rg; blk0 < G; blk0 += RG * U) {
            float4 v[U];
#pragma unroll
            for (int k = 0; k < U; ++k) {
                const int blk = blk0 + RG * k;
                v[k] = blk < G ? *reinterpret_cast<const float4 *>(partials + ((size_t)blk * NB + b) * H + col)
                               : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int k = 0; k < U; ++k) { s.x += v[k].x; s.y += v[k].y; s.z += v[k].z; s.w += v[k].w; }
        }
    }
    red[rg][q] = s;
    __syncthreads();
    if (rg == 0 && col < H) {
        for (int k = 1; k < RG; ++k) {
            const float4 v = red[k][q];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        T *o = out + (size_t)b * H + col;
        o[0] = from_float<T>(s.x); o[1] = from_float<T>(s.y);
        o[2] = from_float<T>(s.z); o[3] = from_float<T>(s.w);
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
constexpr int kMaxLds = 160 * 1024;
#ifndef ST_REDUCE_CW
#define ST_REDUCE_CW 8
#endif
constexpr int kReduceCW = ST_REDUCE_CW;   // threads per row of the reduce kernel: 4 * CW columns per block

struct MlpLaunch {
    const void *x; int B; int H;
    const void *gate, *up, *down;
    int n; const int *n_dev; int n_hint;
    void *out; void *combined; long ldc;
    float *partials;
    int act, has_gate;
    hipStream_t stream;
    int G;
};

template <typename T, int NB, int RB, int CPT, int TPB, bool DB>
static int launch_inst(const MlpLaunch &a, int b0, int bcount)
{
    const int chunks = a.H / Elem<T>::kVec;
    int gs_log2 = 6;
    while ((1 << gs_log2) < chunks && (1 << gs_log2) < TPB) ++gs_log2;
    ST_REQUIRE(chunks <= CPT * (1 << gs_log2), "st_mlp_forward: hidden size %d too large for this dtype", a.H);
    const int ngrp = TPB >> gs_log2;
    const size_t lds = (size_t)(ngrp - 1) * NB * a.H * 4;
    ST_REQUIRE(lds <= (size_t)kMaxLds - 8192, "st_mlp_forward: H=%d needs %zu bytes of LDS", a.H, lds);
    auto kern = mlp_decode_kernel<T, NB, RB, CPT, TPB, DB>;
    static std::atomic<bool> attr_set{false};   // (setting the attribute twice from two threads is harmless)
    if (!attr_set.load(std::memory_order_acquire)) {
        ST_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   kMaxLds - 8192));
        attr_set.store(true, std::memory_order_release);
    }
    const T *x = static_cast<const T *>(a.x) + (size_t)b0 * a.H;
    T *comb = a.combined ? static_cast<T *>(a.combined) + (size_t)b0 * a.ldc : nullptr;
    ST_REQUIRE(a.G <= 0xffff, "st_mlp_forward: %d blocks", a.G);
    const int launch_word = a.G | (gs_log2 << 16) | ((a.has_gate ? 1 : 0) << 20) | (bcount << 24);
    const int n_spec = a.n_dev ? (a.n_hint < a.n ? a.n_hint : a.n) : a.n;   // rows requested ahead of the device's count
    {
        ProfScope ps(ST_K_MLP_DECODE, a.stream);
        ST_LAUNCH(ps, kern, dim3(a.G), dim3(TPB), lds, a.stream, x, static_cast<const T *>(a.gate),
                  static_cast<const T *>(a.up), static_cast<const T *>(a.down), a.n_dev, a.H, launch_word, n_spec,
                  a.n, comb, a.ldc, a.partials, a.act);
    }
    ST_HIP(hipGetLastError());
    T *out = static_cast<T *>(a.out) + (size_t)b0 * a.H;
    {
        ProfScope ps(ST_K_MLP_REDUCE, a.stream);
        ST_LAUNCH(ps, (mlp_reduce_kernel<T, kReduceCW>), dim3((a.H + 4 * kReduceCW - 1) / (4 * kReduceCW), bcount),
                  dim3(kReduceThreads), 0, a.stream, a.partials, a.G, NB, bcount, a.H, out);
    }
    ST_HIP(hipGetLastError());
    return ST_OK;
}

static int env_int(const char *name)
{
    const char *v = getenv(name);
    return v ? atoi(v) : 0;
}

// The launch shape trades registers for loads in flight: measured on MI355X,
// about 12-18 outstanding 16-byte loads per thread with 16 waves per CU
// streams fastest; many more per thread is slower.  RB is the depth of ONE of
// the two register buffers.
template <typename T, int NB> static int launch_one(const MlpLaunch &a, int b0, int bcount)
{
    const int chunks = a.H / Elem<T>::kVec;
    ST_REQUIRE(chunks <= 2048, "st_mlp_forward: hidden size %d too large for this dtype (max %d)", a.H,
               2048 * Elem<T>::kVec);
    if constexpr (NB == 1) {
        if (chunks > 1024) return launch_inst<T, 1, 3, 2, 1024, false>(a, b0, bcount);
        // (512-thread blocks, 3 / 4 / 12 rows in flight and double-buffered row batches were all measured
        // slower for one row of x)
        // (the rows in flight do not change which rows a group sums or in which order: when the expected count
        // gives a group seven rows, one batch of seven beats a batch of six followed by a batch of one; likewise
        // wherever sevens need fewer batches than sixes)
        if constexpr (Elem<T>::kBytes == 2) {
            int gs_log2 = 6;
            while ((1 << gs_log2) < chunks && (1 << gs_log2) < 1024) ++gs_log2;
            const int ngrp = 1024 >> gs_log2, expect = a.n_dev ? (a.n_hint < a.n ? a.n_hint : a.n) : a.n;
            const int rpg = ((expect + a.G - 1) / a.G + ngrp - 1) / ngrp;
            if ((rpg + 6) / 7 < (rpg + 5) / 6) return launch_inst<T, 1, 7, 1, 1024, false>(a, b0, bcount);   // 7, 13, 14, ...
        }
        return launch_inst<T, 1, DecodeRows<T>::value, 1, 1024, false>(a, b0, bcount);
    } else if constexpr (NB == 2) {
        return launch_inst<T, 2, 2, 1, 1024, true>(a, b0, bcount);
    } else if constexpr (NB == 4) {
        if (chunks > 512) return launch_inst<T, 4, 1, 2, 512, true>(a, b0, bcount);
        return launch_inst<T, 4, 3, 1, 512, true>(a, b0, bcount);
    } else {
        return launch_inst<T, 8, 2, 1, 512, true>(a, b0, bcount);  // chunks <= 512 only (see launch_nb)
    }
}

template <typename T> static int launch_nb(const MlpLaunch &a)
{
    const int chunks = a.H / Elem<T>::kVec;
    int b0 = 0;
    while (b0 < a.B) {
        const int left = a.B - b0;
        int rc;
        if (chunks > 1024) {  // very wide rows: one row of x per pass
            rc = launch_one<T, 1>(a, b0, 1);
            b0 += 1;
        } else if (left >= 5 && chunks <= 512) {
            rc = launch_one<T, 8>(a, b0, left < 8 ? left : 8);
            b0 += 8;
        } else if (left >= 3) {
            rc = launch_one<T, 4>(a, b0, left < 4 ? left : 4);
            b0 += 4;
        } else if (left == 2) {
            rc = launch_one<T, 2>(a, b0, 2);
            b0 += 2;
        } else {
            rc = launch_one<T, 1>(a, b0, 1);
            b0 += 1;
        }
        if (rc != ST_OK) return rc;
    }
    return ST_OK;
}

constexpr int kMlpMaxBatchPerLaunch = 8;

// Rows of x from which the MFMA batch kernels take over from the streaming kernel: three (with two the
// streaming kernel measures the same as they do, and it is the arithmetic of the fused update + decode kernel
// for two rows, whose result has to equal update followed by forward).  ST_MLP_BATCH_MIN overrides; 32 or more
// switches the batch kernels off.
int batch_min_rows()
{
    static const int v = [] { const int m = env_int("ST_MLP_BATCH_MIN"); return m >= 2 ? m : 3; }();
    return v;
}

// Blocks per launch: one per CU by default; ST_MLP_GMULT (1..4) multiplies it.
int mlp_grid()
{
    static const int mult = [] { const int m = env_int("ST_MLP_GMULT"); return m >= 1 && m <= 4 ? m : 1; }();
    return device_cu_count() * mult;
}

int launch_mlp_reduce(int dtype, const float *partials, int G, int NB, int bcount, int H, void *out,
                      hipStream_t stream)
{
    ProfScope ps(ST_K_MLP_REDUCE, stream);
    constexpr int CW = kReduceCW;
    const dim3 grid((H + 4 * CW - 1) / (4 * CW), bcount);
    if (dtype == ST_F32)
        ST_LAUNCH(ps, (mlp_reduce_kernel<float, CW>), grid, dim3(kReduceThreads), 0, stream, partials, G, NB, bcount, H,
                           static_cast<float *>(out));
    else if (dtype == ST_F16)
        ST_LAUNCH(ps, (mlp_reduce_kernel<f16_t, CW>), grid, dim3(kReduceThreads), 0, stream, partials, G, NB, bcount, H,
                           static_cast<f16_t *>(out));
    else
        ST_LAUNCH(ps, (mlp_reduce_kernel<bf16_t, CW>), grid, dim3(kReduceThreads), 0, stream, partials, G, NB, bcount, H,
                           static_cast<bf16_t *>(out));
    ST_HIP(hipGetLastError());
    return ST_OK;
}

// Argument checks shared by the MLP entry points (everything but the workspace size).
static int check_mlp_args(const char *who, const void *x, int64_t B, int64_t H, const void *gate_rows,
                          const void *up_rows, const void *down_rows, int64_t n, const void *out, const void *combined,
                          int64_t ldc, const void *workspace, int act, int dtype, int has_gate, bool f64_ok = false)
{
    ST_REQUIRE(x && up_rows && down_rows && out && workspace, "%s: null pointer", who);
    ST_REQUIRE(!has_gate || gate_rows, "%s: has_gate set but gate_rows is null", who);
    ST_REQUIRE(B >= 1 && B <= 4096, "%s: B=%lld out of range [1,4096]", who, (long long)B);
    ST_REQUIRE(n >= 0 && n <= (1 << 24), "%s: n=%lld out of range", who, (long long)n);
    ST_REQUIRE(act >= ST_ACT_RELU && act <= ST_ACT_IDENTITY, "%s: unknown activation %d", who, act);
    ST_REQUIRE((dtype >= ST_F32 && dtype <= ST_BF16) || (f64_ok && dtype == ST_F64), "%s: unknown dtype %d%s", who, dtype,
               dtype == ST_F64 ? " (double precision: st_mlp_forward only)" : "");
    const int esz = dtype == ST_F64 ? 8 : dtype == ST_F32 ? 4 : 2;
    ST_REQUIRE(H >= 1 && (H * esz) % 16 == 0, "%s: H=%lld rows are not 16-byte multiples", who, (long long)H);
    ST_REQUIRE(!combined || ldc >= (has_gate ? 2 * n : n), "%s: ldc=%lld too small for n=%lld", who, (long long)ldc,
               (long long)n);
    const uintptr_t align = (uintptr_t)x | (uintptr_t)gate_rows | (uintptr_t)up_rows | (uintptr_t)down_rows |
                            (uintptr_t)workspace;
    ST_REQUIRE((align & 15) == 0, "%s: pointers must be 16-byte aligned", who);
    return ST_OK;
}

// The streaming decode kernel (+ its reduce) on `workspace`, which holds at least
// blocks x min(B, 8) x H fp32 partial rows.  Allocates nothing.
static int mlp_forward_decode(const void *x, int64_t B, int64_t H, const void *gate_rows, const void *up_rows,
                              const void *down_rows, int64_t n, const int32_t *n_dev, int64_t n_hint, void *out,
                              void *combined, int64_t ldc, void *workspace, int64_t workspace_bytes, int act,
                              int dtype, int has_gate, void *stream, const char *who)
{
    const int rc = check_mlp_args(who, x, B, H, gate_rows, up_rows, down_rows, n, out, combined, ldc, workspace, act,
                                  dtype, has_gate);
    if (rc != ST_OK) return rc;
    MlpLaunch a;
    a.G = mlp_grid();
    const int64_t rows = B <= 2 ? B : (B <= 4 ? 4 : kMlpMaxBatchPerLaunch);   // rows of x per pass (launch_nb)
    ST_REQUIRE(workspace_bytes >= (int64_t)a.G * rows * H * 4, "%s: workspace too small (%lld < %lld)", who,
               (long long)workspace_bytes, (long long)((int64_t)a.G * rows * H * 4));
    a.x = x; a.B = (int)B; a.H = (int)H;
    a.gate = gate_rows; a.up = up_rows; a.down = down_rows;
    a.n = (int)n; a.n_dev = n_dev;
    a.n_hint = (int)(n_hint < 0 ? 0 : (n_hint > n ? n : n_hint));
    a.out = out; a.combined = combined; a.ldc = (long)ldc;
    a.partials = static_cast<float *>(workspace);
    a.act = act; a.has_gate = has_gate ? 1 : 0;
    a.stream = static_cast<hipStream_t>(stream);
    switch (dtype) {
    case ST_F32: return launch_nb<float>(a);
    case ST_F16: return launch_nb<f16_t>(a);
    default: return launch_nb<bf16_t>(a);
    }
}

}  // namespace st

// Device address of `scratch` on the current device, resolved once per device.
static int static_scratch_ptr(void **out)
{
    static std::mutex mu;
    static void *ptrs[64] = {nullptr};
    int dev = 0;
    ST_HIP(hipGetDevice(&dev));
    ST_REQUIRE(dev >= 0 && dev < 64, "st_mlp_forward_static: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(mu);
    if (!ptrs[dev]) {
        void *p = nullptr;
        ST_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(st::scratch)));   // the copy of the array on the current device
        ST_REQUIRE(p != nullptr, "st_mlp_forward_static: hipGetSymbolAddress returned a null address");
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return ST_OK;
}

extern "C" int64_t st_mlp_static_scratch_bytes(void) { return (int64_t)st::kStaticScratchBytes; }

extern "C" int st_mlp_forward_static(const void *x, int64_t B, int64_t H, const void *gate_rows, const void *up_rows,
                                     const void *down_rows, int64_t n, const int32_t *n_dev, int64_t n_hint,
                                     void *out, void *combined, int64_t ldc, int act, int dtype, int has_gate,
                                     void *stream)
{
    using namespace st;
    ST_REQUIRE(B >= 1 && B <= 2, "st_mlp_forward_static: B=%lld outside [1,2] (use st_mlp_forward with a workspace)",
               (long long)B);
    ST_REQUIRE(H >= 1, "st_mlp_forward_static: H=%lld", (long long)H);
    // what the streaming kernel writes: one fp32 row per block and row of x
    const int64_t need = (int64_t)mlp_grid() * B * H * 4;
    ST_REQUIRE(need <= (int64_t)kStaticScratchBytes,
               "st_mlp_forward_static: %lld blocks x %lld rows x H=%lld needs %lld bytes of scratch, the static buffer "
               "holds %lld", (long long)mlp_grid(), (long long)B, (long long)H, (long long)need,
               (long long)kStaticScratchBytes);
    void *ws = nullptr;
    const int rc = static_scratch_ptr(&ws);
    if (rc != ST_OK) return rc;
    return mlp_forward_decode(x, B, H, gate_rows, up_rows, down_rows, n, n_dev, n_hint, out, combined, ldc, ws,
                              (int64_t)kStaticScratchBytes, act, dtype, has_gate, stream, "st_mlp_forward_static");
}

extern "C" int64_t st_mlp_workspace_bytes(int64_t B, int64_t H, int64_t n)
{
    const int64_t G = st::mlp_grid();
    int64_t decode = G * st::kMlpMaxBatchPerLaunch * H * 4;
    if (B >= st::batch_min_rows() && B <= st::kBatchMaxRows) {   // dtype is not known here: size for both paths
        const int64_t batch = st::batch_workspace_bytes(H, n);
        decode = batch > decode ? batch : decode;
    }
    if (B < st::kPrefillMinRows) return decode;
    const int64_t prefill = st::prefill_workspace_bytes(B, H, n);
    return prefill > decode ? prefill : decode;
}

extern "C" int st_mlp_forward(const void *x, int64_t B, int64_t H, const void *gate_rows, const void *up_rows,
                              const void *down_rows, int64_t n, const int32_t *n_dev, int64_t n_hint, void *out,
                              void *combined, int64_t ldc, void *workspace, int64_t workspace_bytes, int act,
                              int dtype, int has_gate, void *stream)
{
    using namespace st;
    const int rc = check_mlp_args("st_mlp_forward", x, B, H, gate_rows, up_rows, down_rows, n, out, combined, ldc,
                                  workspace, act, dtype, has_gate, true);
    if (rc != ST_OK) return rc;
    if (dtype == ST_F64) {
        ST_REQUIRE(workspace_bytes >= f64_workspace_bytes(B, H, n),
                   "st_mlp_forward: workspace too small for double precision (%lld < %lld, st_mlp_f64_workspace_bytes)",
                   (long long)workspace_bytes, (long long)f64_workspace_bytes(B, H, n));
        return launch_f64(x, (int)B, (int)H, gate_rows, up_rows, down_rows, (int)n, n_dev, out, combined, (long)ldc,
                          workspace, act, has_gate ? 1 : 0, static_cast<hipStream_t>(stream));
    }
    ST_REQUIRE(workspace_bytes >= st_mlp_workspace_bytes(B, H, n), "st_mlp_forward: workspace too small (%lld < %lld)",
               (long long)workspace_bytes, (long long)st_mlp_workspace_bytes(B, H, n));

    const bool batch = B >= batch_min_rows() && B <= kBatchMaxRows && batch_supported(dtype, (int)H);
    if (B >= kPrefillMinRows && !batch && dtype != ST_F32 && H % 128 == 0 && n >= 1)
        return launch_prefill(dtype, x, (int)B, (int)H, gate_rows, up_rows, down_rows, (int)n, n_dev, out, combined,
                              (long)ldc, workspace, act, has_gate ? 1 : 0, static_cast<hipStream_t>(stream));

    if (batch)
        return launch_batch(dtype, x, (int)B, (int)H, gate_rows, up_rows, down_rows, (int)n, n_dev, out, combined,
                            (long)ldc, workspace, act, has_gate ? 1 : 0, static_cast<hipStream_t>(stream));

    return mlp_forward_decode(x, B, H, gate_rows, up_rows, down_rows, n, n_dev, n_hint, out, combined, ldc, workspace,
                              workspace_bytes, act, dtype, has_gate, stream, "st_mlp_forward");
}
