// Sparse MLP over the active set for a small batch of rows of x (3 <= B <= 32):
// still bound by the HBM stream of the active rows, but with B rows of x the
// multiply-adds no longer fit beside it on the vector ALUs, so they go to the
// matrix cores (fp16 / bf16 MFMA 16x16x32, fp32 accumulate).  16 rows of x form
// the N (kernel 1) / M (kernel 2) dimension of one tile; both kernels take up
// to two such tiles in one pass over the weights.
//
//   kernel 1  h[b][j] = act(x_b . gate_j) * (x_b . up_j)
//             one block per CU owns a contiguous range of active rows and works
//             through it in tiles of 32 rows.  The 8 waves split the hidden
//             dimension: weight fragments go from HBM straight into MFMA
//             operand registers (16 rows x 64 bytes per load instruction, which
//             streams as fast as fully coalesced loads on this chip), x comes
//             from LDS (one tile) or from registers that hold the wave's slice
//             of the hidden dimension (two tiles), and the 8 partial tiles are
//             summed through LDS.
//   kernel 2  out[b][:] = sum_j h[b][j] * down_j[:]
//             K runs down the rows of the packed down matrix, so the operand
//             has to be transposed: blocks own (column group, row split), each
//             wave stages 32 rows x 64 columns in LDS and reads the fragment
//             with the transposing LDS load.  Split-K partial rows are summed in a fixed order
//             by kernel 3 (mlp_reduce_kernel).
// Unlike a per-CU fused kernel this writes no per-CU partial [B,H] rows (which
// would cost B * 3 MB of extra traffic); h (B * n elements) is the only
// intermediate.
//
// Same contraction as sparse_mlp_forward_cpu
// (sparse_transformers/csrc/sparse_mlp_op.cpp:151-161,181-186) and
// SkipMLP._forward_sparse_weight_cache (src/modeling_skip.py:114-117).
#include "st_mfma.h"

#include <atomic>

namespace st {

constexpr int kBtThreads = 512;
constexpr int kBtWaves = kBtThreads / kWave;
constexpr int kBtRows = 16;                      // rows of x per MFMA tile (kernel 1 takes two tiles per pass)
constexpr int kBtXPad = 8;                       // padding elements per x row in LDS (spreads the banks)
constexpr int kBtTile = 32;                      // active rows per tile / K per MFMA in kernel 2
constexpr int kBtRedFloats = kBtWaves * 2 * 256; // kernel 1: 8 waves x (g,u) x 16x16, one subtile at a time
constexpr int kBtStagePitch = 72;                // kernel 2: elements per staged row (64 + 8 pad)
constexpr int kBtStageBytes = kBtTile * kBtStagePitch * 2;

typedef short bt_v4i16_t __attribute__((ext_vector_type(4)));

// Orders this wave's LDS traffic for the compiler (the hardware executes one wave's LDS operations in order).
__device__ __forceinline__ void wave_lds_fence()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// ---------------------------------------------------------------------------
// kernel 1.  KSW = MFMA k-steps per wave = H / 256; HG = gated; NT = tiles of 16 rows of x (1 or 2).
// h is written as hbuf[b * ldh + row] for all 16 NT b (rows of x past B are zeros).
// ---------------------------------------------------------------------------
template <typename T, int KSW, bool HG, int NT>
__global__ __launch_bounds__(kBtThreads) void batch_gateup_kernel(
    const T *__restrict__ x, int B, int G, const T *__restrict__ gate, const T *__restrict__ up, int n_host,
    const int *__restrict__ n_dev, T *__restrict__ hbuf, int ldh, T *__restrict__ combined, long ldc, int act)
{
    constexpr int H = KSW * 256;
    // k-steps of weight loads in flight per wave (the x fragments take 4 NT KSW registers)
    constexpr int DEPTH = NT == 1 ? (KSW < 6 ? KSW : 6) : (KSW > 12 ? 4 : 5);
    // One tile of x (NT == 1) is staged in LDS by the whole block with full-line loads and read from there;
    // two tiles do not fit, so every wave keeps the fragments of its K slice in registers (measured 0.4-1.2 us
    // slower per launch for one tile: a fragment load touches 16 half lines).
    constexpr bool XREG = NT > 1;
    constexpr int XP = H + kBtXPad;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T *xs = reinterpret_cast<T *>(lds_raw);                                                      // [16][XP]
    float *red = reinterpret_cast<float *>(lds_raw + (XREG ? 0 : (size_t)kBtRows * XP * 2));     // [NT][8][2][4][64]

    const int tid = threadIdx.x, lane = tid & (kWave - 1), w = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int blk = blockIdx.x;  // G: the grid's size, an argument so that it arrives preloaded

    const int n = device_count(n_host, n_dev);
    const int R = (n + G - 1) / G;             // rows per block
    const int row0 = blk * R;
    const int jcount = n - row0 < R ? n - row0 : R;
    if (jcount <= 0) return;

    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    const int ntile = (jcount + kBtTile - 1) / kBtTile;

    // this lane's weight rows in the two 16-row subtiles of tile t
    bool v0, v1;
    size_t o0, o1;
    auto setup = [&](int t) __attribute__((always_inline)) {
        const int j0 = t * kBtTile + r, j1 = j0 + 16;
        v0 = j0 < jcount; v1 = j1 < jcount;
        o0 = (size_t)(row0 + (v0 ? j0 : 0)) * H + 8 * q + 32 * w;
        o1 = (size_t)(row0 + (v1 ? j1 : 0)) * H + 8 * q + 32 * w;
    };
    uint4 g0[KSW], u0[KSW], g1[KSW], u1[KSW];
    auto issue = [&](int j) __attribute__((always_inline)) {
        const int col = 256 * j;   // step j of wave w covers columns 32 * (8 j + w) ..
        u0[j] = zero4; u1[j] = zero4;
        if (HG) { g0[j] = zero4; g1[j] = zero4; }
        if (v0) {                  // lanes without a row request nothing
            u0[j] = ld16(up + o0 + col);
            if (HG) g0[j] = ld16(gate + o0 + col);
        }
        if (v1) {
            u1[j] = ld16(up + o1 + col);
            if (HG) g1[j] = ld16(gate + o1 + col);
        }
    };

    // x is requested first, then the first weight loads.  XREG: lane (r, q) of wave w holds columns
    // 256 j + 32 w + 8 q .. + 7 of row 16 t + r (rows past B are zeros).
    const T *xfrag = xs + (size_t)r * XP + 8 * q + 32 * w;
    uint4 xr[XREG ? NT : 1][XREG ? KSW : 1];
    if constexpr (XREG) {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const bool ok = 16 * t + r < B;
            const T *xp = x + (size_t)(ok ? 16 * t + r : 0) * H + 8 * q + 32 * w;
#pragma unroll
            for (int j = 0; j < KSW; ++j) {
                xr[t][j] = zero4;
                if (ok) xr[t][j] = ld16(xp + 256 * j);
            }
        }
        setup(0);
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) issue(j);
    } else {
        // 16 rows x H/8 chunks = KSW chunks per thread; staging x waits for x alone
        constexpr int chunks = H / 8;
        uint4 xv[KSW];
#pragma unroll
        for (int i = 0; i < KSW; ++i) {
            const int idx = tid + kBtThreads * i;
            const int b = idx / chunks, c = idx - b * chunks;
            xv[i] = zero4;
            if (b < B) xv[i] = ld16(x + (size_t)b * H + c * 8);
        }
        setup(0);
#pragma unroll
        for (int j = 0; j < DEPTH; ++j) issue(j);
#pragma unroll
        for (int i = 0; i < KSW; ++i) {
            const int idx = tid + kBtThreads * i;
            const int b = idx / chunks, c = idx - b * chunks;
            *reinterpret_cast<uint4 *>(xs + (size_t)b * XP + c * 8) = xv[i];
        }
        __syncthreads();
    }

    for (int t = 0; t < ntile; ++t) {
        if (t > 0) {
            setup(t);
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) issue(j);
        }

        f32x4_t dg0[NT], du0[NT], dg1[NT], du1[NT];
#pragma unroll
        for (int xt = 0; xt < NT; ++xt) {
            dg0[xt] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            du0[xt] = dg0[xt]; dg1[xt] = dg0[xt]; du1[xt] = dg0[xt];
        }
#pragma unroll
        for (int j = 0; j < KSW; ++j) {
#pragma unroll
            for (int xt = 0; xt < NT; ++xt) {
                uint4 xf;
                if constexpr (XREG) xf = xr[xt][j];
                else xf = *reinterpret_cast<const uint4 *>(xfrag + 256 * j);
                du0[xt] = Mfma<T>::run(u0[j], xf, du0[xt]);
                if (HG) dg0[xt] = Mfma<T>::run(g0[j], xf, dg0[xt]);
                du1[xt] = Mfma<T>::run(u1[j], xf, du1[xt]);
                if (HG) dg1[xt] = Mfma<T>::run(g1[j], xf, dg1[xt]);
            }
            if (j + DEPTH < KSW) issue(j + DEPTH);
        }

        // sum the 8 waves' partial tiles, one 16-row subtile at a time: red[xt][w][g|u][e][lane]
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s == 1 && jcount - t * kBtTile <= 16) break;   // the second subtile is empty (uniform)
#pragma unroll
            for (int xt = 0; xt < NT; ++xt) {
                float *mine = red + (size_t)(xt * kBtWaves + w) * 512 + lane;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (HG) mine[e * 64] = s == 0 ? dg0[xt][e] : dg1[xt][e];
                    mine[(4 + e) * 64] = s == 0 ? du0[xt][e] : du1[xt][e];
                }
            }
            __syncthreads();
            if (tid < 256 * NT) {
                // thread -> one element of a 16x16 tile: D register e of D lane dl of x tile xt
                const int xt = tid >> 8, e = (tid >> 6) & 3, dl = tid & 63;
                float sg = 0.f, su = 0.f;
#pragma unroll
                for (int ww = 0; ww < kBtWaves; ++ww) {
                    if (HG) sg += red[(size_t)(xt * kBtWaves + ww) * 512 + e * 64 + dl];
                    su += red[(size_t)(xt * kBtWaves + ww) * 512 + (4 + e) * 64 + dl];
                }
                const int j = t * kBtTile + 16 * s + 4 * (dl >> 4) + e;   // D rows are 4 * (lane / 16) + e
                const int b = 16 * xt + (dl & 15);
                if (j < jcount) {
                    const float hv = HG ? activate(sg, act) * su : activate(su, act);
                    const int row = row0 + j;
                    hbuf[(size_t)b * ldh + row] = from_float<T>(hv);
                    if (combined && b < B) {
                        combined[(size_t)b * ldc + row] = from_float<T>(hv);
                        if (HG) combined[(size_t)b * ldc + n + row] = from_float<T>(su);
                    }
                }
            }
            __syncthreads();   // red is rewritten by the next subtile / tile
        }
    }
}

// ---------------------------------------------------------------------------
// kernel 1 for any hidden size that is a multiple of 256 (the hidden sizes above have instantiations of their own):
// the number of k-steps per wave is a run-time value, the weight fragments go through a ring of kBtRing slots, and
// the x fragments come from LDS while a 16-row tile of x fits there (XLDS: H <= 4096) or straight from memory
// (hits in L1 / L2 after the first tile) beyond.  One tile of 16 rows of x per pass; same block / tile / wave
// decomposition and the same sums as batch_gateup_kernel<T, KSW, HG, 1>.
// ---------------------------------------------------------------------------
constexpr int kBtRing = 4;

template <typename T, bool HG, bool XLDS>
__global__ __launch_bounds__(kBtThreads) void batch_gateup_anyh_kernel(
    const T *__restrict__ x, int B, int H, int G, const T *__restrict__ gate, const T *__restrict__ up, int n_host,
    const int *__restrict__ n_dev, T *__restrict__ hbuf, int ldh, T *__restrict__ combined, long ldc, int act)
{
    const int KSW = H / 256, XP = H + kBtXPad;
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T *xs = reinterpret_cast<T *>(lds_raw);                                                      // [16][XP] (XLDS)
    float *red = reinterpret_cast<float *>(lds_raw + (XLDS ? (size_t)kBtRows * XP * 2 : 0));     // [8][2][4][64]

    const int tid = threadIdx.x, lane = tid & (kWave - 1), w = tid >> 6;
    const int r = lane & 15, q = lane >> 4;
    const int blk = blockIdx.x;  // G: the grid's size, an argument so that it arrives preloaded

    const int n = device_count(n_host, n_dev);
    const int R = (n + G - 1) / G;
    const int row0 = blk * R;
    const int jcount = n - row0 < R ? n - row0 : R;
    if (jcount <= 0) return;

    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    const int ntile = (jcount + kBtTile - 1) / kBtTile;

    bool v0, v1;
    size_t o0, o1;
    auto setup = [&](int t) __attribute__((always_inline)) {
        const int j0 = t * kBtTile + r, j1 = j0 + 16;
        v0 = j0 < jcount; v1 = j1 < jcount;
        o0 = (size_t)(row0 + (v0 ? j0 : 0)) * H + 8 * q + 32 * w;
        o1 = (size_t)(row0 + (v1 ? j1 : 0)) * H + 8 * q + 32 * w;
    };
    uint4 g0[kBtRing], u0[kBtRing], g1[kBtRing], u1[kBtRing];
    auto issue = [&](int slot, int j) __attribute__((always_inline)) {
        const int col = 256 * j;
        u0[slot] = zero4; u1[slot] = zero4;
        if (HG) { g0[slot] = zero4; g1[slot] = zero4; }
        if (v0) {
            u0[slot] = ld16(up + o0 + col);
            if (HG) g0[slot] = ld16(gate + o0 + col);
        }
        if (v1) {
            u1[slot] = ld16(up + o1 + col);
            if (HG) g1[slot] = ld16(gate + o1 + col);
        }
    };

    const bool xrow_ok = r < B;
    const T *xglob = x + (size_t)(xrow_ok ? r : 0) * H + 8 * q + 32 * w;
    const T *xfrag = xs + (size_t)r * XP + 8 * q + 32 * w;
    if constexpr (XLDS) {   // stage the tile of x: 16 rows x H/8 chunks, KSW chunks per thread
        const int chunks = H / 8;
        for (int i = 0; i < KSW; ++i) {
            const int idx = tid + kBtThreads * i;
            const int b = idx / chunks, c = idx - b * chunks;
            uint4 xv = zero4;
            if (b < B) xv = ld16(x + (size_t)b * H + c * 8);
            *reinterpret_cast<uint4 *>(xs + (size_t)b * XP + c * 8) = xv;
        }
    }
    setup(0);
#pragma unroll
    for (int sl = 0; sl < kBtRing; ++sl)
        if (sl < KSW) issue(sl, sl);
    if constexpr (XLDS) __syncthreads();

    for (int t = 0; t < ntile; ++t) {
        if (t > 0) {
            setup(t);
#pragma unroll
            for (int sl = 0; sl < kBtRing; ++sl)
                if (sl < KSW) issue(sl, sl);
        }
        f32x4_t dg0 = f32x4_t{0.f, 0.f, 0.f, 0.f}, du0 = dg0, dg1 = dg0, du1 = dg0;
        for (int jb = 0; jb < KSW; jb += kBtRing) {
#pragma unroll
            for (int sl = 0; sl < kBtRing; ++sl) {
                const int j = jb + sl;
                if (j < KSW) {   // uniform
                    uint4 xf;
                    if constexpr (XLDS) xf = *reinterpret_cast<const uint4 *>(xfrag + 256 * j);
                    else xf = xrow_ok ? ld16(xglob + 256 * j) : zero4;
                    du0 = Mfma<T>::run(u0[sl], xf, du0);
                    if (HG) dg0 = Mfma<T>::run(g0[sl], xf, dg0);
                    du1 = Mfma<T>::run(u1[sl], xf, du1);
                    if (HG) dg1 = Mfma<T>::run(g1[sl], xf, dg1);
                    if (j + kBtRing < KSW) issue(sl, j + kBtRing);
                }
            }
        }
        // sum the 8 waves' partial tiles, one 16-row subtile at a time (as in batch_gateup_kernel)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
            if (s == 1 && jcount - t * kBtTile <= 16) break;
            float *mine = red + (size_t)w * 512 + lane;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (HG) mine[e * 64] = s == 0 ? dg0[e] : dg1[e];
                mine[(4 + e) * 64] = s == 0 ? du0[e] : du1[e];
            }
            __syncthreads();
            if (tid < 256) {
                const int e = (tid >> 6) & 3, dl = tid & 63;
                float sg = 0.f, su = 0.f;
#pragma unroll
                for (int ww = 0; ww < kBtWaves; ++ww) {
                    if (HG) sg += red[(size_t)ww * 512 + e * 64 + dl];
                    su += red[(size_t)ww * 512 + (4 + e) * 64 + dl];
                }
                const int j = t * kBtTile + 16 * s + 4 * (dl >> 4) + e;
                const int b = dl & 15;
                if (j < jcount) {
                    const float hv = HG ? activate(sg, act) * su : activate(su, act);
                    const int row = row0 + j;
                    hbuf[(size_t)b * ldh + row] = from_float<T>(hv);
                    if (combined && b < B) {
                        combined[(size_t)b * ldc + row] = from_float<T>(hv);
                        if (HG) combined[(size_t)b * ldc + n + row] = from_float<T>(su);
                    }
                }
            }
            __syncthreads();
        }
    }
}

// ---------------------------------------------------------------------------
// kernel 2.  Block = (column group cg, row split rs); NP = 64-column pieces per
// block; NX = tiles of 16 rows of x.  partial[(rs * 16 NX + b) * H + col], fp32.
// ---------------------------------------------------------------------------
template <typename T, int NP, int NX>
__global__ __launch_bounds__(kBtThreads) void batch_down_kernel(
    const T *__restrict__ hbuf, int ldh, int B, const T *__restrict__ down, int H, int n_host,
    const int *__restrict__ n_dev, float *__restrict__ partial, int CG, int RS)
{
    constexpr int NT = NP * 4;   // 16-column tiles per block
    extern __shared__ __align__(16) unsigned char lds_raw[];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), w = tid >> 6;
    const int c16 = lane & 15, q = lane >> 4;
    const int cg = blockIdx.x % CG, rs = blockIdx.x / CG;
    const int col0 = cg * NP * 64;

    const int n = device_count(n_host, n_dev);
    const int NC = (n + kBtTile - 1) / kBtTile;        // chunks of 32 rows
    const int CPS = (NC + RS - 1) / RS;
    const int c_begin = rs * CPS;
    const int c_end = c_begin + CPS < NC ? c_begin + CPS : NC;

    T *stage = reinterpret_cast<T *>(lds_raw + (size_t)w * kBtStageBytes);

    f32x4_t acc[NX][NT];
#pragma unroll
    for (int t = 0; t < NX; ++t)
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[t][i] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    struct Chunk { uint4 d[NP][4]; uint2 hlo[NX], hhi[NX]; };
    // 8 rows x 128 bytes per load instruction
    auto load_chunk = [&](Chunk &k, int c) __attribute__((always_inline)) {
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            int row = c * kBtTile + (lane >> 3) + 8 * kk;
            row = row < n ? row : n - 1;   // clamped rows meet zeros of h
            const T *rp = down + (size_t)row * H + col0 + 8 * (lane & 7);
#pragma unroll
            for (int p = 0; p < NP; ++p) k.d[p][kk] = ld16(rp + 64 * p);
        }
        // h fragment: k-slots 0..3 <-> rows 4q..4q+3, slots 4..7 <-> rows 16+4q..16+4q+3 of the chunk
#pragma unroll
        for (int t = 0; t < NX; ++t) {
            const T *hp = hbuf + (size_t)(16 * t + c16) * ldh + c * kBtTile + 4 * q;
            k.hlo[t] = *reinterpret_cast<const uint2 *>(hp);
            k.hhi[t] = *reinterpret_cast<const uint2 *>(hp + 16);
        }
    };
    auto process = [&](const Chunk &k, int c) __attribute__((always_inline)) {
        uint4 hf[NX];
#pragma unroll
        for (int t = 0; t < NX; ++t) {
            uint32_t a[4] = {k.hlo[t].x, k.hlo[t].y, k.hhi[t].x, k.hhi[t].y};
            if (c * kBtTile + kBtTile > n) {   // rows past the count hold nothing defined
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int rlo = c * kBtTile + (i < 2 ? 4 * q + 2 * i : 16 + 4 * q + 2 * (i - 2));
                    if (rlo >= n) a[i] = 0u;
                    else if (rlo + 1 >= n) a[i] &= 0xffffu;
                }
            }
            hf[t] = make_uint4(a[0], a[1], a[2], a[3]);
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            wave_lds_fence();   // the previous piece's reads come first
#pragma unroll
            for (int kk = 0; kk < 4; ++kk)
                *reinterpret_cast<uint4 *>(stage + ((lane >> 3) + 8 * kk) * kBtStagePitch + 8 * (lane & 7)) = k.d[p][kk];
            wave_lds_fence();
#pragma unroll
            for (int ct = 0; ct < 4; ++ct) {
                // transposing LDS read: in its group of 16 lanes, lane j hands in four columns of row j / 4 and
                // lane i receives column i of the four rows (rows 4q.. and 16 + 4q.. of the staged piece)
                const uint16_t *sp = reinterpret_cast<const uint16_t *>(stage) +
                                     (4 * q + (c16 >> 2)) * kBtStagePitch + 16 * ct + 4 * (c16 & 3);
                const bt_v4i16_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) bt_v4i16_t *)sp);
                const bt_v4i16_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) bt_v4i16_t *)(sp + 16 * kBtStagePitch));
                const uint4 bf = make_uint4((uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16),
                                            (uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16),
                                            (uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16),
                                            (uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16));
#pragma unroll
                for (int t = 0; t < NX; ++t) acc[t][p * 4 + ct] = Mfma<T>::run(hf[t], bf, acc[t][p * 4 + ct]);
            }
        }
    };

    Chunk ka, kb;
    int c = c_begin + w;
    if (c < c_end) load_chunk(ka, c);
    while (c < c_end) {
        int cn = c + kBtWaves;
        if (cn < c_end) load_chunk(kb, cn);
        process(ka, c);
        c = cn;
        if (c >= c_end) break;
        cn = c + kBtWaves;
        if (cn < c_end) load_chunk(ka, cn);
        process(kb, c);
        c = cn;
    }

    // sum the 8 waves' accumulators through LDS (reuses the staging area), one tile of x at a time
#pragma unroll
    for (int t = 0; t < NX; ++t) {
        __syncthreads();
        float *red = reinterpret_cast<float *>(lds_raw);   // [8][NT][4][64]
#pragma unroll
        for (int i = 0; i < NT; ++i)
#pragma unroll
            for (int e = 0; e < 4; ++e) red[((size_t)(w * NT + i) * 4 + e) * 64 + lane] = acc[t][i][e];
        __syncthreads();
#pragma unroll
        for (int m = 0; m < NT * 256 / kBtThreads; ++m) {
            const int idx = tid + kBtThreads * m;
            float s = 0.f;
#pragma unroll
            for (int ww = 0; ww < kBtWaves; ++ww) s += red[(size_t)ww * NT * 256 + idx];
            const int tile = idx >> 8, e = (idx >> 6) & 3, dl = idx & 63;
            const int b = 16 * t + 4 * (dl >> 4) + e;   // D rows are the rows of x
            if (b < B) partial[((size_t)rs * (kBtRows * NX) + b) * H + col0 + 16 * tile + (dl & 15)] = s;
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct BatchShape { int ksw, np, cg, rs; bool special; };
constexpr int kBtMaxH = 16384;

static bool batch_shape(int H, BatchShape &s)
{
    if (H % 256 != 0 || H < 256 || H > kBtMaxH) return false;
    s.ksw = H / 256;
    s.special = s.ksw == 8 || s.ksw == 12 || s.ksw == 16;   // hidden sizes with kernels instantiated for them
    const int pieces = H / 64;
    s.np = pieces % 3 == 0 ? 3 : 2;   // 4 pieces with two chunks in flight would not fit the register file
    s.cg = pieces / s.np;
    s.rs = device_cu_count() / s.cg;
    if (s.rs < 1) s.rs = 1;
    if (s.rs > 32) s.rs = 32;
    return true;
}

bool batch_supported(int dtype, int H)
{
    BatchShape s;
    return dtype != ST_F32 && batch_shape(H, s);
}

static int64_t batch_ldh(int64_t n) { return (n + kBtTile - 1) / kBtTile * kBtTile; }

int64_t batch_workspace_bytes(int64_t H, int64_t n)
{
    const int64_t hh = ((int64_t)2 * kBtRows * batch_ldh(n) * 2 + 255) & ~(int64_t)255;   // h of up to 32 rows of x
    return hh + (int64_t)32 * kBtRows * H * 4;
}

template <typename T, int KSW, bool HG, int NT>
static int launch_gateup(const T *x, int B, const T *gate, const T *up, int n, const int *n_dev, T *hbuf, int ldh,
                         T *comb, long ldc, int act, hipStream_t stream)
{
    auto kern = batch_gateup_kernel<T, KSW, HG, NT>;
    const size_t lds = (NT == 1 ? (size_t)kBtRows * (KSW * 256 + kBtXPad) * 2 : 0) + (size_t)NT * kBtRedFloats * 4;
    static std::atomic<bool> attr_set{false};   // (setting the attribute twice from two threads is harmless)
    if (!attr_set.load(std::memory_order_acquire)) {
        ST_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds));
        attr_set.store(true, std::memory_order_release);
    }
    ProfScope ps(ST_K_MLP_BATCH_GATEUP, stream);
    const int G = device_cu_count();
    ST_LAUNCH(ps, kern, dim3(G), dim3(kBtThreads), lds, stream, x, B, G, gate, up, n, n_dev, hbuf,
                       ldh, comb, ldc, act);
    return ST_OK;
}

template <typename T, bool HG>
static int launch_gateup_anyh(const T *x, int B, int H, const T *gate, const T *up, int n, const int *n_dev, T *hbuf,
                              int ldh, T *comb, long ldc, int act, hipStream_t stream)
{
    const bool xlds = H <= 4096;
    const size_t lds = (xlds ? (size_t)kBtRows * (H + kBtXPad) * 2 : 0) + (size_t)kBtRedFloats * 4;
    ProfScope ps(ST_K_MLP_BATCH_GATEUP, stream);
    const int G = device_cu_count();
    if (xlds) {
        auto kern = batch_gateup_anyh_kernel<T, HG, true>;
        const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), 152 * 1024);
        if (rc != ST_OK) return rc;
        ST_LAUNCH(ps, kern, dim3(G), dim3(kBtThreads), lds, stream, x, B, H, G, gate, up, n, n_dev, hbuf,
                  ldh, comb, ldc, act);
    } else {
        auto kern = batch_gateup_anyh_kernel<T, HG, false>;
        ST_LAUNCH(ps, kern, dim3(G), dim3(kBtThreads), lds, stream, x, B, H, G, gate, up, n, n_dev, hbuf,
                  ldh, comb, ldc, act);
    }
    return ST_OK;
}

template <typename T, int NP, int NX>
static int launch_down(const T *hbuf, int ldh, int B, const T *down, int H, int n, const int *n_dev, float *partial,
                       int cg, int rs, hipStream_t stream)
{
    auto kern = batch_down_kernel<T, NP, NX>;
    const size_t red = (size_t)kBtWaves * NP * 4 * 256 * 4, stage = (size_t)kBtWaves * kBtStageBytes;
    const size_t lds = red > stage ? red : stage;
    static std::atomic<bool> attr_set{false};   // (setting the attribute twice from two threads is harmless)
    if (!attr_set.load(std::memory_order_acquire)) {
        ST_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                   (int)lds));
        attr_set.store(true, std::memory_order_release);
    }
    ProfScope ps(ST_K_MLP_BATCH_DOWN, stream);
    ST_LAUNCH(ps, kern, dim3(cg * rs), dim3(kBtThreads), lds, stream, hbuf, ldh, B, down, H, n, n_dev, partial, cg, rs);
    return ST_OK;
}

template <typename T>
static int launch_batch_t(const void *x_, int B, int H, const void *gate_, const void *up_, const void *down_, int n,
                          const int *n_dev, void *out_, void *comb_, long ldc, void *workspace, int act, int has_gate,
                          hipStream_t stream)
{
    BatchShape s;
    ST_REQUIRE(batch_shape(H, s), "st_mlp_forward: hidden size %d is not supported by the batch kernels", H);
    const int ldh = (int)batch_ldh(n);
    T *hbuf = static_cast<T *>(workspace);
    const int64_t hh_bytes = ((int64_t)2 * kBtRows * ldh * 2 + 255) & ~(int64_t)255;
    float *partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + hh_bytes);
    const T *gate = static_cast<const T *>(gate_), *up = static_cast<const T *>(up_);
    const T *down = static_cast<const T *>(down_);
    // gate / up: one pass over the weights per 32 rows of x (16 with the kernel for other hidden sizes); down: one per 16
    const int pass_rows = s.special ? 2 * kBtRows : kBtRows;
    for (int b0 = 0; b0 < B; b0 += pass_rows) {
        const int bc = B - b0 < pass_rows ? B - b0 : pass_rows;
        const T *x = static_cast<const T *>(x_) + (size_t)b0 * H;
        T *comb = comb_ ? static_cast<T *>(comb_) + (size_t)b0 * ldc : nullptr;
        int rc;
#define ST_BT_GATEUP(KSW)                                                                                              \
    rc = bc > kBtRows                                                                                                 \
             ? (has_gate ? launch_gateup<T, KSW, true, 2>(x, bc, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream)   \
                         : launch_gateup<T, KSW, false, 2>(x, bc, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream)) \
             : (has_gate ? launch_gateup<T, KSW, true, 1>(x, bc, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream)   \
                         : launch_gateup<T, KSW, false, 1>(x, bc, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream))
        if (!s.special)
            rc = has_gate ? launch_gateup_anyh<T, true>(x, bc, H, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream)
                          : launch_gateup_anyh<T, false>(x, bc, H, gate, up, n, n_dev, hbuf, ldh, comb, ldc, act, stream);
        else if (s.ksw == 8) ST_BT_GATEUP(8);
        else if (s.ksw == 12) ST_BT_GATEUP(12);
        else ST_BT_GATEUP(16);
#undef ST_BT_GATEUP
        if (rc != ST_OK) return rc;
        ST_HIP(hipGetLastError());
        // kernel 2 takes both tiles of x in one pass with two 64-column pieces per block (three would not leave
        // registers for a second set of accumulators); kernel 3 sums the row splits' partial rows
        // [rs][16 or 32][H] in a fixed order (the streaming kernels' reduce kernel)
        T *out = static_cast<T *>(out_) + (size_t)b0 * H;
        int rs = s.rs, nbrows = kBtRows;
        if (bc > kBtRows) {
            const int cg = H / 128;
            rs = device_cu_count() / cg;
            rs = rs < 1 ? 1 : (rs > 16 ? 16 : rs);
            nbrows = 2 * kBtRows;
            rc = launch_down<T, 2, 2>(hbuf, ldh, bc, down, H, n, n_dev, partial, cg, rs, stream);
        } else {
            rc = s.np == 3 ? launch_down<T, 3, 1>(hbuf, ldh, bc, down, H, n, n_dev, partial, s.cg, s.rs, stream)
                           : launch_down<T, 2, 1>(hbuf, ldh, bc, down, H, n, n_dev, partial, s.cg, s.rs, stream);
        }
        if (rc != ST_OK) return rc;
        ST_HIP(hipGetLastError());
        rc = launch_mlp_reduce(sizeof(T) == 2 && __is_same(T, f16_t) ? ST_F16 : ST_BF16, partial, rs, nbrows, bc, H, out,
                               stream);
        if (rc != ST_OK) return rc;
    }
    return ST_OK;
}

int launch_batch(int dtype, const void *x, int B, int H, const void *gate, const void *up, const void *down, int n,
                 const int *n_dev, void *out, void *comb, long ldc, void *workspace, int act, int has_gate,
                 hipStream_t stream)
{
    if (dtype == ST_F16)
        return launch_batch_t<f16_t>(x, B, H, gate, up, down, n, n_dev, out, comb, ldc, workspace, act, has_gate, stream);
    return launch_batch_t<bf16_t>(x, B, H, gate, up, down, n, n_dev, out, comb, ldc, workspace, act, has_gate, stream);
}

}  // namespace st
