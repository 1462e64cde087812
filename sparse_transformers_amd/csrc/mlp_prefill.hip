// Sparse MLP over the active set for many rows of x (prefill / large batch):
// a dense contraction, so it runs on the matrix cores (fp16 / bf16 MFMA
// 16x16x32, fp32 accumulate).
//
//   kernel 1  Hh[M,n] = act(X Wg^T) * (X Wu^T)       X [M,H], Wg/Wu [n,H]
//             both operands are K-contiguous, tiles go global -> LDS as is;
//             gate and up share the X fragments, the activation is applied
//             to the accumulators before Hh is written
//   kernel 2  Out[M,H] = Hh[M,n] Wd[n,H]              Wd rows are the packed
//             down columns, i.e. K runs down the rows: the tile sits in LDS
//             as [k][column] and the fragments are read with the
//             transposing LDS load (ds_read_b64_tr_b16)
// Each kernel has two forms.  The first (kernel 1: 64 or 128 rows of x by 32 or 64 active rows of gate and of up
// per block; kernel 2: block tile 128 x 128 with split-K) has waves of 64 x 64 and K stages of 64 through two LDS
// buffers with the following stages' global loads held in registers, one barrier per stage; it serves the shapes
// whose tiles do not fill the chip.  The wide form (256 x 128 block tiles, waves of 128 x 64 whose K the two waves
// of a SIMD share, operands loaded global -> LDS directly through three buffers) takes over when they do.
//
// The reference only runs the sparse path for decode (src/modeling_skip.py:236);
// this is the same contraction as sparse_mlp_forward_cpu
// (sparse_transformers/csrc/sparse_mlp_op.cpp:151-161) for B > 1 rows.
#include <type_traits>

#include "st_mfma.h"

namespace st {

constexpr int kPfThreads = 256;
constexpr int kPfBM = 128;   // rows of x per block
constexpr int kPfBN = 128;   // output columns per block (kernel 1: 64 gate + 64 up rows)
constexpr int kPfBK = 128;   // columns of Hh are padded to a multiple of this

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

// ---------------------------------------------------------------------------
// epilogues shared by the two forms of each kernel
// ---------------------------------------------------------------------------
// D[m][j] of a 16 x 16 MFMA block: a lane holds rows 4 q + e (e = 0..3) of column l16.
//
// Kernel 1: the activation on a wave's 64 x 16 JN gate / up sums, and the product stored into Hh (and `comb`).
// Columns n .. n_pad are written as zeros so that kernel 2 can run whole K stages.  The results go through a tile
// of the wave's own in LDS (`stg`, 64 rows of 16 JN + 8 elements; the stage buffers are free by then) and leave as
// whole 16-byte chunks, 64 bytes of a row per four lanes; storing every element by itself took 5.2 us of the 57
// the kernel ran.
template <typename T, bool HG, int JN, int ACT>
__device__ __forceinline__ void pf_store_hidden_as(const f32x4_t (&ag)[4][JN], const f32x4_t (&au)[4][JN], T *stg,
                                                   int lane, int mrow0, int colw, int M, int n, int n_pad, T *Hh,
                                                   long ldh, T *comb, long ldc)
{
    constexpr int kSP = 16 * JN + 8;   // elements per staged row (16-byte multiple, spreads the banks)
    const int l16 = lane & 15, q = lane >> 4;
    const bool comb16 = comb && ldc % 8 == 0 && (reinterpret_cast<uintptr_t>(comb) & 15) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j) {
            const int col = colw + 16 * j + l16;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float hv = 0.f;
                if (col < n) hv = HG ? activate_fast(ag[i][j][e], ACT) * au[i][j][e] : activate_fast(au[i][j][e], ACT);
                stg[(16 * i + 4 * q + e) * kSP + 16 * j + l16] = from_float<T>(hv);
            }
        }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int c = 0; c < 2 * JN; ++c) {
        const int idx = lane + 64 * c, row = idx / (2 * JN), ch = idx % (2 * JN);
        const int m = mrow0 + row, col0 = colw + 8 * ch;
        if (m < M && col0 < n_pad) {
            const uint4 v = *reinterpret_cast<const uint4 *>(stg + row * kSP + 8 * ch);
            *reinterpret_cast<uint4 *>(Hh + (size_t)m * ldh + col0) = v;
            if (comb16 && col0 + 8 <= n) {
                *reinterpret_cast<uint4 *>(comb + (size_t)m * ldc + col0) = v;
            } else if (comb) {
                const T *sv = stg + row * kSP + 8 * ch;
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (col0 + k < n) comb[(size_t)m * ldc + col0 + k] = sv[k];
            }
        }
    }
}

// One copy per activation, chosen once per block: with the activation switched per element the whole kernel was
// 4 us slower (all five bodies live in the loop's register budget).
template <typename T, bool HG, int JN>
__device__ __forceinline__ void pf_store_hidden(int act, const f32x4_t (&ag)[4][JN], const f32x4_t (&au)[4][JN], T *stg,
                                                int lane, int mrow0, int colw, int M, int n, int n_pad, T *Hh, long ldh,
                                                T *comb, long ldc)
{
    switch (act) {
    case ST_ACT_RELU: pf_store_hidden_as<T, HG, JN, ST_ACT_RELU>(ag, au, stg, lane, mrow0, colw, M, n, n_pad, Hh, ldh, comb, ldc); break;
    case ST_ACT_SILU: pf_store_hidden_as<T, HG, JN, ST_ACT_SILU>(ag, au, stg, lane, mrow0, colw, M, n, n_pad, Hh, ldh, comb, ldc); break;
    case ST_ACT_GELU_TANH: pf_store_hidden_as<T, HG, JN, ST_ACT_GELU_TANH>(ag, au, stg, lane, mrow0, colw, M, n, n_pad, Hh, ldh, comb, ldc); break;
    case ST_ACT_SIGMOID: pf_store_hidden_as<T, HG, JN, ST_ACT_SIGMOID>(ag, au, stg, lane, mrow0, colw, M, n, n_pad, Hh, ldh, comb, ldc); break;
    default: pf_store_hidden_as<T, HG, JN, ST_ACT_IDENTITY>(ag, au, stg, lane, mrow0, colw, M, n, n_pad, Hh, ldh, comb, ldc); break;
    }
}

// Kernel 2: a wave's 64 x 64 sums, either straight into Out (no K split) or as fp32 partial sums of split z through
// a tile of the wave's own in LDS (`stg`, 64 rows of 68 floats), 256 bytes of a row per 16 lanes.
constexpr int kPfStgF = 64 + 4;   // floats per staged row
template <typename T>
__device__ __forceinline__ void pf_store_out(const f32x4_t (&f)[4][4], float *stg, int lane, int mrow0, int colw, int M,
                                             int H, T *Out, float *partial_z)
{
    const int l16 = lane & 15, q = lane >> 4;
    if (!partial_z) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int col = colw + 16 * j + l16;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = mrow0 + 16 * i + 4 * q + e;
                    if (m < M && col < H) Out[(size_t)m * H + col] = from_float<T>(f[i][j][e]);
                }
            }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 4; ++e) stg[(16 * i + 4 * q + e) * kPfStgF + 16 * j + l16] = f[i][j][e];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int c = 0; c < 16; ++c) {
        const int row = 4 * c + q, m = mrow0 + row, col = colw + 4 * l16;
        if (m < M && col < H)
            *reinterpret_cast<float4 *>(partial_z + (size_t)m * H + col) =
                *reinterpret_cast<const float4 *>(stg + row * kPfStgF + 4 * l16);
    }
}

// ---------------------------------------------------------------------------
// kernel 1: gate / up projections + activation
// ---------------------------------------------------------------------------
// K stages of 64 (one 128-byte line of every row), two LDS buffers and NS register sets: stage s is
// requested from memory NS stages ahead, goes from registers into the LDS buffer of its parity while the
// MFMAs of stage s - 1 run, and costs one barrier.  BM rows of x by 64 (or 32) gate + as many up rows per
// block, 2 BM threads, every wave a 64 x (32 + 32) (or 64 x (16 + 16)) tile.  HG: gated.
constexpr int kPfBK1 = 64;
constexpr int kPfCh1 = kPfBK1 / 8;   // 16-byte chunks per row and stage
constexpr int kPfLd1 = kPfCh1;       // LDS row stride in 16-byte units: 128 bytes, no padding
// K-contiguous tiles in LDS: chunk c of row r sits at position c ^ pf_swz(r).  Rows are 128 bytes, so even and
// odd rows take the two halves of the 64 banks and the XOR spreads eight row pairs over a half: the 16 rows of a
// fragment read (one chunk each) and the two rows of a 16-lane store (eight chunks each) both meet every bank
// once.  (With 144-byte rows the reads were free of conflicts but the stores were not: a third of the LDS
// cycles of kernel 1 were bank conflicts.)
__device__ __forceinline__ int pf_swz(int row) { return (row >> 1) & 7; }

// KS = 2 or 4: as many groups of 2 BM threads share a tile, each runs its part of K through LDS buffers of its own,
// and the other groups' accumulators are added to the first's through LDS at the end.
// JN = 16-row tiles of gate and of up per wave: 2 (64 rows of each per block) or, to make more blocks out of
// few rows, 1 (32 rows of each).
template <typename T, bool HG, int BM, int NS, int KS, int JN>
__global__ __launch_bounds__(2 * BM * KS) void prefill_gateup_kernel(const T *__restrict__ X,
                                                                     const T *__restrict__ gate,
                                                                     const T *__restrict__ up,
                                                                     const int *__restrict__ n_dev, int M, int H,
                                                                     int n_host, int jt, int mt,
                                                                     T *__restrict__ Hh, long ldh,
                                                                     T *__restrict__ comb, long ldc, int act)
{
    // (operands, sizes and the tile grid first: the first 14 dwords of the arguments are in scalar registers when the
    // wave starts; what only the epilogue needs arrives by a load)
    constexpr int kThreads = 2 * BM;                     // per K group
    constexpr int kWR = 32 * JN;                         // rows of gate and of up per block
    constexpr int kRows = BM + (HG ? 2 : 1) * kWR;       // LDS rows of one buffer: x, gate, up
    __shared__ uint4 lds[KS * 2 * kRows * kPfLd1];

    const int n = device_count(n_host, n_dev);
    const int n_pad = (n + kPfBK - 1) / kPfBK * kPfBK;  // kernel 2 runs whole K stages over Hh
    const int tile = xcd_tile_id(blockIdx.x, jt * mt);   // row tiles of x fastest: they share the weight rows
    if (tile < 0) return;
    const int j0 = (tile / mt) * kWR, m0 = (tile % mt) * BM;
    if (j0 >= n_pad) return;
    ST_TL(0);
    const int kh = KS > 1 ? threadIdx.x / kThreads : 0;  // K group
    const int tid = threadIdx.x - kh * kThreads, lane = tid & 63, wave = tid >> 6;
    uint4 (*sX)[kRows][kPfLd1] = reinterpret_cast<uint4 (*)[kRows][kPfLd1]>(lds + (size_t)kh * 2 * kRows * kPfLd1);
    constexpr int kGRow = BM, kURow = BM + (HG ? kWR : 0);   // first LDS row of the gate and of the up tile
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;

    // global -> register staging: thread owns chunk `ch` of rows r0 + kRowStep i
    const int ch = tid & (kPfCh1 - 1), r0 = tid / kPfCh1;
    constexpr int kRowStep = kThreads / kPfCh1;
    static_assert(kRowStep % 16 == 0 && BM % 16 == 0, "the swizzle of a thread's rows must not depend on i");
    const int chs = ch ^ pf_swz(r0);               // where this thread's chunk sits in its LDS rows
    const int fsw = pf_swz(l16);                   // the same for the rows this lane reads fragments from
    constexpr int kXL = BM / kRowStep;             // loads for x
    constexpr int kWL = kWR / kRowStep;            // loads for gate and for up

    f32x4_t ag[4][JN], au[4][JN];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < JN; ++j) {
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
    struct Stage { uint4 x[kXL], g[kWL], u[kWL]; };
    Stage R[NS];
    const int nk = H / kPfBK1 / KS;   // stages of this K group (H is a multiple of 128)
    const int kbase = kh * nk * kPfBK1, klast = (nk - 1) * kPfBK1;
    auto gload = [&](Stage &st, int stage) __attribute__((always_inline)) {
        const int k0 = kbase + (stage * kPfBK1 <= klast ? stage * kPfBK1 : klast);   // past the end: a harmless repeat
#pragma unroll
        for (int i = 0; i < kXL; ++i) st.x[i] = ld16(X + xoff[i] + k0);
#pragma unroll
        for (int i = 0; i < kWL; ++i) {
            st.u[i] = ld16(up + woff[i] + k0);
            if (HG) st.g[i] = ld16(gate + woff[i] + k0);
        }
    };
    auto sstore = [&](const Stage &st, int b) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < kXL; ++i) sX[b][r0 + kRowStep * i][chs] = st.x[i];
#pragma unroll
        for (int i = 0; i < kWL; ++i) {
            if (HG) sX[b][kGRow + r0 + kRowStep * i][chs] = st.g[i];
            sX[b][kURow + r0 + kRowStep * i][chs] = st.u[i];
        }
    };
    // fragments of one k step (32 of K): x rows of this wave, its gate and up rows
    struct Frag { uint4 a[4], g[JN], u[JN]; };
    Frag F0, F1;
    auto lfrag = [&](Frag &F, int b, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) F.a[i] = sX[b][64 * wm + 16 * i + l16][(4 * kb + q) ^ fsw];
#pragma unroll
        for (int j = 0; j < JN; ++j) {
            if (HG) F.g[j] = sX[b][kGRow + 16 * JN * wn + 16 * j + l16][(4 * kb + q) ^ fsw];
            F.u[j] = sX[b][kURow + 16 * JN * wn + 16 * j + l16][(4 * kb + q) ^ fsw];
        }
    };
    auto mm = [&](const Frag &F) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < JN; ++j) {
                au[i][j] = Mfma<T>::run(F.a[i], F.u[j], au[i][j]);
                if (HG) ag[i][j] = Mfma<T>::run(F.a[i], F.g[j], ag[i][j]);
            }
    };
    // One stage: the second k step's fragments are requested before the MFMAs of the first, the next stage's first
    // fragments (after the barrier that completes its LDS buffer) before the MFMAs of the second.  The scheduling
    // barriers keep that order: left alone, the compiler sinks every fragment read to just before its first use.
    auto stage = [&](int u, bool store, int next) __attribute__((always_inline)) {
        lfrag(F1, u & 1, 1);
        __builtin_amdgcn_sched_barrier(0);
        mm(F0);
        __builtin_amdgcn_sched_barrier(0);
        if (store) sstore(R[(u + 1) % NS], (u + 1) & 1);
        __syncthreads();
        lfrag(F0, (u + 1) & 1, 0);
        __builtin_amdgcn_sched_barrier(0);
        mm(F1);
        __builtin_amdgcn_sched_barrier(0);
        gload(R[(u + 1) % NS], next);
    };

#pragma unroll
    for (int s = 0; s < NS; ++s) gload(R[s], s);
    sstore(R[0], 0);
    __syncthreads();
    gload(R[0], NS);
    lfrag(F0, 0, 0);
    ST_TL(1);
    // stage s = base + u lives in LDS buffer u & 1 and came through register set u % NS (2 NS divides base).
    // Whole groups of 2 NS stages run without any checks (as straight-line code the compiler interleaves the
    // loads, LDS stores and MFMAs; with a test per stage the kernel is a quarter slower); the last group tests.
    int base = 0;
    for (; base + 2 * NS < nk; base += 2 * NS) {
#pragma unroll
        for (int u = 0; u < 2 * NS; ++u) stage(u, true, base + u + 1 + NS);
    }
    ST_TL(2);
#pragma unroll
    for (int u = 0; u < 2 * NS; ++u) {
        const int s = base + u;
        if (s >= nk) break;
        stage(u, s + 1 < nk, s + 1 + NS);
    }
    ST_TL(3);

    constexpr int kWG = kThreads / 64;                      // waves per K group
    constexpr int kRedWave = (HG ? 8 : 4) * JN * 256;       // floats one wave hands over
    if constexpr (KS > 1) {
        // the stage loops end with a barrier, so the buffers are free: the other groups hand their sums over
        float *red = reinterpret_cast<float *>(lds) + ((size_t)(kh > 0 ? kh - 1 : 0) * kWG + wave) * kRedWave + lane;
        if (kh > 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < JN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        red[((i * JN + j) * 4 + e) * 64] = au[i][j][e];
                        if (HG) red[((4 * JN + i * JN + j) * 4 + e) * 64] = ag[i][j][e];
                    }
        }
        __syncthreads();
        if (kh > 0) return;
#pragma unroll
        for (int g = 0; g < KS - 1; ++g)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < JN; ++j)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        au[i][j][e] += red[(size_t)g * kWG * kRedWave + ((i * JN + j) * 4 + e) * 64];
                        if (HG) ag[i][j][e] += red[(size_t)g * kWG * kRedWave + ((4 * JN + i * JN + j) * 4 + e) * 64];
                    }
    }

    // the stage loops end with a barrier, so the buffers are free for the epilogue's tiles
    constexpr int kSP = 16 * JN + 8;
    constexpr size_t kStgOff = KS > 1 ? (size_t)(KS - 1) * kWG * kRedWave * (4 / sizeof(T)) : 0;   // past the sums
    static_assert((kStgOff + (size_t)kWG * 64 * kSP) * sizeof(T) <= sizeof(lds), "epilogue tiles exceed the stage buffers");
    T *stg = reinterpret_cast<T *>(lds) + kStgOff + (size_t)wave * 64 * kSP;
    pf_store_hidden<T, HG, JN>(act, ag, au, stg, lane, m0 + 64 * wm, j0 + 16 * JN * wn, M, n, n_pad, Hh, ldh, comb, ldc);
    ST_TL(4);
}

// ---------------------------------------------------------------------------
// kernel 1, wide form: 256 rows of x by 64 gate + 64 up rows per block, operands straight into LDS
// ---------------------------------------------------------------------------
// The form above reads 8 KB of fragments from LDS for every 16 MFMAs of a wave (64 x 64 wave tiles), which at
// the LDS's ~110 bytes per clock takes as long as the MFMAs themselves.  Here a wave owns a 128 x (32 + 32)
// tile (12 KB of fragments per 32 MFMAs) and the two waves of a SIMD share one tile: wave kh takes the
// kh-th 32 of every 64-wide K stage into accumulators of its own, and the pair is summed through LDS once
// at the end.  The operands do not pass through registers on their way in: every wave issues its share of a
// stage as 1 KB global -> LDS loads (lane i's 16 bytes land at base + 16 i, so the lane asks for the chunk
// that belongs at that place of the swizzled row), two stages ahead into the third of three LDS buffers,
// and only waits -- on the count of its own outstanding loads -- before the stage's barrier.
constexpr int kPwBM = 256, kPwWR = 64, kPwThreads = 512, kPwBufs = 3;

// s_waitcnt immediate: vmcnt in bits 3:0 (and 15:14), expcnt 6:4 left at "no wait", lgkmcnt 11:8 = 0
#define ST_WAIT_VM_LGKM0(vm) __builtin_amdgcn_s_waitcnt(((vm) & 15) | (7 << 4) | (0 << 8) | (((vm) >> 4) << 14))

// 64 lanes x 16 bytes from `base + off` (uniform base, per-lane byte offset) to the 1 KB of LDS at byte address
// `dst` (uniform), lane i's 16 bytes at dst + 16 i.  The instruction takes the LDS address from M0; the compiler is not
// told about M0 (it is a reserved register for inline assembly), so its value is put back, and the write of M0 is
// followed by the wait state the instruction needs before it may read it.
__device__ __forceinline__ void pf_load_to_lds(unsigned dst, unsigned off, const char *base)
{
    unsigned keep;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %2, %3\n\ts_mov_b32 m0, %0"
                 : "=&s"(keep)
                 : "s"(dst), "v"(off), "s"(base)
                 : "memory");
}

template <typename T, bool HG>
__global__ __launch_bounds__(kPwThreads) void prefill_gateup_wide_kernel(const T *__restrict__ X,
                                                                         const T *__restrict__ gate,
                                                                         const T *__restrict__ up,
                                                                         const int *__restrict__ n_dev, int M, int H,
                                                                         int n_host, int jt, int mt,
                                                                         T *__restrict__ Hh, long ldh,
                                                                         T *__restrict__ comb, long ldc, int act)
{
    constexpr int kRows = kPwBM + (HG ? 2 : 1) * kPwWR;   // LDS rows of one buffer: x, gate, up
    constexpr int kBuf = kRows * kPfLd1;                  // 16-byte units per buffer
    constexpr int kDma = kRows / 64;                      // 1 KB loads per wave and stage
    constexpr int kGRow = kPwBM, kURow = kPwBM + (HG ? kPwWR : 0);
    __shared__ uint4 lds[kPwBufs * kBuf];

    const int n = device_count(n_host, n_dev);
    const int n_pad = (n + kPfBK - 1) / kPfBK * kPfBK;
    const int tile = xcd_tile_id(blockIdx.x, jt * mt);
    if (tile < 0) return;
    const int j0 = (tile / mt) * kPwWR, m0 = (tile % mt) * kPwBM;
    if (j0 >= n_pad) return;
    ST_TL(0);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kh = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const int fsw = pf_swz(l16);

    // the wave's loads of a stage: load j fills LDS rows 8 L .. 8 L + 7 (L = kDma wave + j), lane i the
    // position i % 8 of row i / 8, which holds chunk (i % 8) ^ pf_swz(row)
    const char *dbase[kDma];
    unsigned doff[kDma];
#pragma unroll
    for (int j = 0; j < kDma; ++j) {
        const int L = wave * kDma + j;
        const int r = 8 * L + (lane >> 3), c = (lane & 7) ^ pf_swz(r);
        int g;
        if (8 * L < kPwBM) {
            g = m0 + r;
            g = g < M ? g : M - 1;
            dbase[j] = reinterpret_cast<const char *>(X);
        } else {
            const bool isg = HG && 8 * L < kURow;
            g = j0 + r - (isg ? kGRow : kURow);
            g = g < n ? g : (n > 0 ? n - 1 : 0);
            dbase[j] = reinterpret_cast<const char *>(isg ? gate : up);
        }
        doff[j] = ((unsigned)g * (unsigned)H + (unsigned)c * 8u) * (unsigned)sizeof(T);
    }
    const int nk = H / kPfBK1;
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // The load is written out as an instruction (pf_load_to_lds): the compiler treats the builtin form as a store to
    // LDS that every later LDS read has to wait for (vmcnt(0) right behind the loads), which is exactly what the
    // three buffers are there to avoid; the waits are placed by hand below.
    auto dma = [&](int stage, int b) __attribute__((always_inline)) {
        const size_t k0 = (size_t)stage * kPfBK1 * sizeof(T);
#pragma unroll
        for (int j = 0; j < kDma; ++j) {
            const unsigned dst = (unsigned)(b * kBuf + (wave * kDma + j) * 64) * 16u + lds_base;
            pf_load_to_lds(dst, doff[j], dbase[j] + k0);
        }
    };

    f32x4_t ag[8][2], au[8][2];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            ag[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
            au[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
        }
    // fragments: the wave's k step of a stage is the kh-th 32 of its 64.  The 128 rows of x go through the MFMAs
    // as four pairs of 16-row fragments, each pair against the wave's two gate and two up fragments.
    struct FragB { uint4 g[2], u[2]; };
    uint4 A[3][2];
    FragB Bc, Bn;
    auto rdA = [&](uint4 (&F)[2], int b, int pair) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
            F[i] = lds[b * kBuf + (128 * wm + 32 * pair + 16 * i + l16) * kPfLd1 + ((4 * kh + q) ^ fsw)];
    };
    auto rdB = [&](FragB &F, int b) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (HG) F.g[j] = lds[b * kBuf + (kGRow + 32 * wn + 16 * j + l16) * kPfLd1 + ((4 * kh + q) ^ fsw)];
            F.u[j] = lds[b * kBuf + (kURow + 32 * wn + 16 * j + l16) * kPfLd1 + ((4 * kh + q) ^ fsw)];
        }
    };
    auto mm = [&](const uint4 (&F)[2], const FragB &W, int pair) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                au[2 * pair + i][j] = Mfma<T>::run(F[i], W.u[j], au[2 * pair + i][j]);
                if (HG) ag[2 * pair + i][j] = Mfma<T>::run(F[i], W.g[j], ag[2 * pair + i][j]);
            }
    };
    // Stage s = base + u (3 divides base) sits in LDS buffer u, its first pair of x fragments in slot u of the
    // ring of three.  The loads of stage s + 2 go out first, into the buffer every wave finished reading before
    // the previous stage's barrier.  Every pair of x fragments is requested before the MFMAs of the pair ahead of
    // it; the next stage's weight fragments and first pair follow the barrier (which follows the wait for this
    // wave's own loads of that stage) and run under the MFMAs of the last pair (past the last stage they read
    // a stale buffer and are not used).  The barrier is the bare instruction: __syncthreads() would also wait
    // for the loads that are meant to stay in flight.
    auto stage = [&](int u, int s) __attribute__((always_inline)) {
        const int x = u, y = (u + 1) % 3, z = (u + 2) % 3;
        const bool load = s + 2 < nk;
        if (load) dma(s + 2, z);
        rdA(A[y], u, 1);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[x], Bc, 0);
        __builtin_amdgcn_sched_barrier(0);
        rdA(A[z], u, 2);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[y], Bc, 1);
        __builtin_amdgcn_sched_barrier(0);
        rdA(A[x], u, 3);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[z], Bc, 2);
        __builtin_amdgcn_sched_barrier(0);
        if (load) ST_WAIT_VM_LGKM0(kDma); else ST_WAIT_VM_LGKM0(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        rdB(Bn, y);
        rdA(A[y], y, 0);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[x], Bc, 3);
        __builtin_amdgcn_sched_barrier(0);
        Bc = Bn;
    };

    dma(0, 0);
    if (nk > 1) dma(1, 1);
    if (nk > 1) ST_WAIT_VM_LGKM0(kDma); else ST_WAIT_VM_LGKM0(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    rdB(Bc, 0);
    rdA(A[0], 0, 0);
    ST_TL(1);
    int base = 0;
    for (; base + 3 <= nk; base += 3) {
        stage(0, base);
        stage(1, base + 1);
        stage(2, base + 2);
    }
    if (base < nk) {
        stage(0, base);
        if (base + 1 < nk) stage(1, base + 1);
    }

    ST_TL(2);
    // The pair's sums: the wave with kh = 0 finishes the first 64 rows of the tile, the other the last 64; each
    // hands the other half of its accumulators over through LDS (all stage buffers are free: the last stage ends
    // behind its barrier with no fragment read outstanding).
    constexpr int kQuads = (HG ? 2 : 1) * 8;   // accumulator quads per lane handed over
    f32x4_t *red = reinterpret_cast<f32x4_t *>(lds);
    f32x4_t fg[4][2], fu[4][2];
    {
        f32x4_t *mine = red + (size_t)wave * kQuads * 64 + lane;
        auto hand = [&](int h) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    mine[(i * 2 + j) * 64] = au[4 * h + i][j];
                    if (HG) mine[(8 + i * 2 + j) * 64] = ag[4 * h + i][j];
                    fu[i][j] = au[4 * (1 - h) + i][j];
                    if (HG) fg[i][j] = ag[4 * (1 - h) + i][j];
                }
        };
        if (kh == 0) hand(1); else hand(0);
    }
    __syncthreads();
    {
        const f32x4_t *other = red + (size_t)(wave ^ 4) * kQuads * 64 + lane;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                fu[i][j] += other[(i * 2 + j) * 64];
                if (HG) fg[i][j] += other[(8 + i * 2 + j) * 64];
            }
    }
    __syncthreads();

    ST_TL(3);
    T *stg = reinterpret_cast<T *>(lds) + (size_t)wave * 64 * (32 + 8);
    pf_store_hidden<T, HG, 2>(act, fg, fu, stg, lane, m0 + 128 * wm + 64 * kh, j0 + 32 * wn, M, n, n_pad, Hh, ldh, comb, ldc);
    ST_TL(4);
}

// ---------------------------------------------------------------------------
// kernel 2: down projection
// ---------------------------------------------------------------------------
// Out[M,H] = Hh[M,n] Wd[n,H].  Wd's rows run along K, so its tile goes to LDS as it is ([k][column], whole
// 16-byte chunks, the two halves of a row swapped on every second group of eight k so that the four
// lane groups of a fragment read meet different banks) and the B fragments come out through the
// transposing LDS read: in a group of 16 lanes, lane j hands in the address of four consecutive columns
// of row j / 4 and lane i receives column i of the four rows.  K stages of 64, two LDS buffers, two
// register sets, block tile 128 x 128, 4 waves of 64 x 64, split-K with a fixed-order reduction.
// H is a multiple of 128 here (the caller routes other widths elsewhere).
constexpr int kPfBK2 = 64;
constexpr int kPfLdB = 18;   // Wd rows in LDS: 16 chunks + 2 of padding (288 bytes)
typedef short pf_v4i16_t __attribute__((ext_vector_type(4)));

template <typename T>
__global__ __launch_bounds__(kPfThreads, 2) void prefill_down_kernel(const T *__restrict__ Hh,
                                                                     const T *__restrict__ Wd,
                                                                     const int *__restrict__ n_dev, long ldh, int M,
                                                                     int H, int n_host, int split_k, int ct, int mt,
                                                                     T *__restrict__ Out, float *__restrict__ partial)
{
    constexpr int NS = 2;
    __shared__ uint4 lds[2 * kPfBM * kPfLd1 + 2 * kPfBK2 * kPfLdB];
    uint4 (*sA)[kPfBM][kPfLd1] = reinterpret_cast<uint4 (*)[kPfBM][kPfLd1]>(lds);
    uint4 (*sB)[kPfBK2][kPfLdB] = reinterpret_cast<uint4 (*)[kPfBK2][kPfLdB]>(lds + 2 * kPfBM * kPfLd1);

    const int n = device_count(n_host, n_dev);
    const int tile = xcd_tile_id(blockIdx.x, ct * mt * split_k);  // row tiles fastest, then column tiles, then splits
    if (tile < 0) return;
    const int z = tile / (ct * mt), c0 = ((tile / mt) % ct) * kPfBN, m0 = (tile % mt) * kPfBM;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);

    // K range of this split, in stages of 64 (Hh is zero-padded to a multiple of 128 columns)
    const int nst_all = (n + kPfBK - 1) / kPfBK * (kPfBK / kPfBK2);
    const int per = (nst_all + split_k - 1) / split_k;
    const int ks0 = z * per, ks1 = (ks0 + per < nst_all) ? ks0 + per : nst_all;
    const int nst = ks1 - ks0;

    // staging: chunk ach of the Hh rows ar0 + 32 i; chunk bch (8 columns) of the Wd rows br0 + 16 i
    const int ach = tid & 7, ar0 = tid >> 3;
    const int bch = tid & 15, br0 = tid >> 4;

    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    int aoff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = m0 + ar0 + 32 * i;
        aoff[i] = (int)((r < M ? r : M - 1) * ldh) + ach * 8;
    }
    const T *wcol = Wd + c0 + 8 * bch;
    const int nlast = n > 0 ? n - 1 : 0;
    struct Stage { uint4 a[4], b[4]; };
    Stage R[NS];
    // Rows of Wd at or beyond n are replaced by zeros (they meet the zero padding of Hh, but stale rows may
    // hold anything, and 0 * inf is not 0); only a split's last stages can reach them.
    auto gload = [&](Stage &st, int s) __attribute__((always_inline)) {
        const int k0 = (s < ks1 ? s : ks1 - 1) * kPfBK2;   // past the end: a harmless repeat
#pragma unroll
        for (int i = 0; i < 4; ++i) st.a[i] = ld16(Hh + aoff[i] + k0);
        if (k0 + kPfBK2 <= n) {
#pragma unroll
            for (int i = 0; i < 4; ++i) st.b[i] = ld16(wcol + (size_t)(k0 + br0 + 16 * i) * H);
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = k0 + br0 + 16 * i;
                st.b[i] = ld16(wcol + (size_t)(r < n ? r : nlast) * H);
                if (r >= n) st.b[i] = zero4;
            }
        }
    };
    auto sstore = [&](const Stage &st, int b) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) sA[b][ar0 + 32 * i][ach ^ pf_swz(ar0)] = st.a[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int k = br0 + 16 * i;
            sB[b][k][bch ^ (8 * ((k >> 3) & 1))] = st.b[i];
        }
    };
    auto mfmas = [&](int b) __attribute__((always_inline)) {
#pragma unroll
        for (int kb = 0; kb < kPfBK2 / 32; ++kb) {
            uint4 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[i] = sA[b][64 * wm + 16 * i + l16][(4 * kb + q) ^ pf_swz(l16)];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                pf_v4i16_t h[2];
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    const int k = 32 * kb + 8 * q + 4 * hh + (l16 >> 2);   // the row this lane hands in
                    const int col = 64 * wn + 16 * j + 4 * (l16 & 3);      // first of its four columns
                    const int chunk = (col >> 3) ^ (8 * ((k >> 3) & 1));
                    const unsigned short *p = reinterpret_cast<const unsigned short *>(&sB[b][k][chunk]) + (col & 7);
                    h[hh] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) pf_v4i16_t *)p);
                }
                fb[j].x = (unsigned short)h[0][0] | ((unsigned)(unsigned short)h[0][1] << 16);
                fb[j].y = (unsigned short)h[0][2] | ((unsigned)(unsigned short)h[0][3] << 16);
                fb[j].z = (unsigned short)h[1][0] | ((unsigned)(unsigned short)h[1][1] << 16);
                fb[j].w = (unsigned short)h[1][2] | ((unsigned)(unsigned short)h[1][3] << 16);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = Mfma<T>::run(fa[i], fb[j], acc[i][j]);
        }
    };

    if (nst > 0) {
#pragma unroll
        for (int s = 0; s < NS; ++s) gload(R[s], ks0 + s);
        sstore(R[0], 0);
        __syncthreads();
        gload(R[0], ks0 + NS);
        // stage ks0 + base + u sits in LDS buffer u & 1 and came through register set u % NS
        int base = 0;
        for (; base + 2 * NS < nst; base += 2 * NS) {   // whole groups: no checks
#pragma unroll
            for (int u = 0; u < 2 * NS; ++u) {
                mfmas(u & 1);
                sstore(R[(u + 1) % NS], (u + 1) & 1);
                __syncthreads();
                gload(R[(u + 1) % NS], ks0 + base + u + 1 + NS);
            }
        }
#pragma unroll
        for (int u = 0; u < 2 * NS; ++u) {
            const int s = base + u;
            if (s >= nst) break;
            mfmas(u & 1);
            if (s + 1 < nst) sstore(R[(u + 1) % NS], (u + 1) & 1);
            __syncthreads();
            gload(R[(u + 1) % NS], ks0 + s + 1 + NS);
        }
    }

    // the stage loop ends with a barrier, so the buffers are free for the waves' tiles
    static_assert(4 * 64 * kPfStgF * 4 <= (int)sizeof(lds), "staging tiles exceed the stage buffers");
    float *stg = reinterpret_cast<float *>(lds) + (size_t)wave * 64 * kPfStgF;
    pf_store_out<T>(acc, stg, lane, m0 + 64 * wm, c0 + 64 * wn, M, H, Out,
                    split_k == 1 ? nullptr : partial + (size_t)z * M * H);
}

// ---------------------------------------------------------------------------
// kernel 2, wide form: 256 rows of Hh by 128 output columns per block and K split, operands straight into LDS
// ---------------------------------------------------------------------------
// The same scheme as prefill_gateup_wide_kernel: waves own 128 x 64 tiles, the two waves of a SIMD share a
// tile (wave kh takes the kh-th 32 of every 64-wide K stage), operands arrive by 1 KB global -> LDS loads
// two stages ahead into three buffers.  Wd's rows run along K and cannot be padded when they are loaded this
// way (a load fills 1 KB of LDS back to back: four rows of 256 bytes), so the 16-byte chunks of row k are
// XORed with 2 (k % 4 + 4 (k / 8 % 2)): the 8 rows x 32 bytes that half a wave hands to the transposing read
// then cover every bank once.
__device__ __forceinline__ int pf_swz_b(int k) { return 2 * ((k & 3) | (((k >> 3) & 1) << 2)); }

template <typename T>
__global__ __launch_bounds__(kPwThreads) void prefill_down_wide_kernel(const T *__restrict__ Hh,
                                                                       const T *__restrict__ Wd,
                                                                       const int *__restrict__ n_dev, long ldh, int M,
                                                                       int H, int n_host, int split_k, int ct, int mt,
                                                                       T *__restrict__ Out,
                                                                       float *__restrict__ partial)
{
    constexpr int kABuf = kPwBM * kPfLd1;             // 16-byte units of the Hh tile of a stage (32 KB)
    constexpr int kBuf = kABuf + kPfBK2 * 16;         // + 64 rows of Wd x 256 bytes (16 KB)
    constexpr int kDma = 6;                           // 1 KB loads per wave and stage
    __shared__ uint4 lds[kPwBufs * kBuf];

    const int n = device_count(n_host, n_dev);
    const int tile = xcd_tile_id(blockIdx.x, ct * mt * split_k);   // row tiles fastest, then column tiles, then splits
    if (tile < 0) return;
    const int z = tile / (ct * mt), c0 = ((tile / mt) % ct) * kPfBN, m0 = (tile % mt) * kPwBM;
    ST_TL(0);
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int kh = wave >> 2, wm = (wave >> 1) & 1, wn = wave & 1;
    const int l16 = lane & 15, q = lane >> 4;
    const int fsw = pf_swz(l16);

    // K range of this split, in stages of 64 (Hh is zero-padded to a multiple of 128 columns)
    const int nst_all = (n + kPfBK - 1) / kPfBK * (kPfBK / kPfBK2);
    const int per = (nst_all + split_k - 1) / split_k;
    const int ks0 = z * per, ks1 = (ks0 + per < nst_all) ? ks0 + per : nst_all;
    const int nst = ks1 - ks0;

    // the wave's loads of a stage: loads L = 6 wave + j; L < 32 fills rows 8 L .. 8 L + 7 of the Hh tile (lane i the
    // position i % 8 of row i / 8), L >= 32 rows 4 (L - 32) .. + 3 of the Wd tile (position i % 16 of row i / 16)
    const char *dbase[kDma];
    unsigned doff[kDma];
    size_t dstep[kDma];
#pragma unroll
    for (int j = 0; j < kDma; ++j) {
        const int L = wave * kDma + j;
        if (L < 32) {
            const int r = 8 * L + (lane >> 3), c = (lane & 7) ^ pf_swz(r);
            int g = m0 + r;
            g = g < M ? g : M - 1;
            dbase[j] = reinterpret_cast<const char *>(Hh) + (size_t)ks0 * kPfBK2 * sizeof(T);
            doff[j] = (unsigned)((size_t)g * ldh * sizeof(T)) + (unsigned)c * 16u;
            dstep[j] = kPfBK2 * sizeof(T);
        } else {
            const int k = 4 * (L - 32) + (lane >> 4), c = (lane & 15) ^ pf_swz_b(k);
            dbase[j] = reinterpret_cast<const char *>(Wd + c0) + (size_t)ks0 * kPfBK2 * H * sizeof(T);
            doff[j] = (unsigned)k * (unsigned)H * (unsigned)sizeof(T) + (unsigned)c * 16u;
            dstep[j] = (size_t)kPfBK2 * H * sizeof(T);
        }
    }
    const unsigned lds_base = (unsigned)(uintptr_t)(__attribute__((address_space(3))) uint4 *)lds;
    // Rows of Wd at or beyond n (they meet the zero padding of Hh, but stale rows may hold anything, and
    // 0 * inf is not 0) are replaced by the last valid row, whose products with the padding are zeros as
    // long as the weights are finite; only a split's last stages can reach them.
    auto dma = [&](int stage, int b, bool check) __attribute__((always_inline)) {
        const bool past = check && (ks0 + stage + 1) * kPfBK2 > n;   // uniform
#pragma unroll
        for (int j = 0; j < kDma; ++j) {
            const unsigned dst = (unsigned)(b * kBuf + (wave * kDma + j) * 64) * 16u + lds_base;
            const char *src = dbase[j] + (size_t)stage * dstep[j];
            unsigned off = doff[j];
            if (past && wave * kDma + j >= 32) {   // uniform: a load of Wd rows
                const int kt = 4 * (wave * kDma + j - 32) + (lane >> 4), k = (ks0 + stage) * kPfBK2 + kt;
                const int kc = k < n ? k : (n > 0 ? n - 1 : 0);
                src = reinterpret_cast<const char *>(Wd + c0);
                off = (unsigned)kc * (unsigned)H * (unsigned)sizeof(T) + (unsigned)((lane & 15) ^ pf_swz_b(kt)) * 16u;
            }
            pf_load_to_lds(dst, off, src);
        }
    };

    f32x4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    uint4 A[3][2], Bc[4], Bn[4];
    auto rdA = [&](uint4 (&F)[2], int b, int pair) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
            F[i] = lds[b * kBuf + (128 * wm + 32 * pair + 16 * i + l16) * kPfLd1 + ((4 * kh + q) ^ fsw)];
    };
    // B fragments through the transposing read: in a group of 16 lanes, lane j hands in the address of four
    // consecutive columns of row j / 4 and lane i receives column i of the four rows
    const int bsw = 2 * ((l16 >> 2) | ((q & 1) << 2));   // pf_swz_b of the rows this lane hands in
    auto rdB = [&](uint4 (&F)[4], int b) __attribute__((always_inline)) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            pf_v4i16_t h[2];
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int k = 32 * kh + 8 * q + 4 * hh + (l16 >> 2);
                const int col = 64 * wn + 16 * j + 4 * (l16 & 3);
                const unsigned short *p16 =
                    reinterpret_cast<const unsigned short *>(&lds[b * kBuf + kABuf + k * 16 + ((col >> 3) ^ bsw)]) + (col & 7);
                h[hh] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) pf_v4i16_t *)p16);
            }
            typedef short v8i16_t __attribute__((ext_vector_type(8)));
            F[j] = __builtin_bit_cast(uint4, (v8i16_t)__builtin_shufflevector(h[0], h[1], 0, 1, 2, 3, 4, 5, 6, 7));
        }
    };
    auto mm = [&](const uint4 (&F)[2], const uint4 (&W)[4], int pair) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[2 * pair + i][j] = Mfma<T>::run(F[i], W[j], acc[2 * pair + i][j]);
    };
    // One stage, as in prefill_gateup_wide_kernel.  `check` is false in the main loop, whose stages all have loads
    // to issue and none of them touches rows of Wd at or beyond n.
    auto stage = [&](int u, int s, bool check) __attribute__((always_inline)) {
        const int x = u, y = (u + 1) % 3, zz = (u + 2) % 3;
        const bool load = !check || s + 2 < nst;
        if (load) dma(s + 2, zz, check);
        rdA(A[y], u, 1);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[x], Bc, 0);
        __builtin_amdgcn_sched_barrier(0);
        rdA(A[zz], u, 2);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[y], Bc, 1);
        __builtin_amdgcn_sched_barrier(0);
        rdA(A[x], u, 3);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[zz], Bc, 2);
        __builtin_amdgcn_sched_barrier(0);
        if (load) ST_WAIT_VM_LGKM0(kDma); else ST_WAIT_VM_LGKM0(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        rdB(Bn, y);
        rdA(A[y], y, 0);
        __builtin_amdgcn_sched_barrier(0);
        mm(A[x], Bc, 3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) Bc[j] = Bn[j];
    };

    if (nst > 0) {
        dma(0, 0, true);
        if (nst > 1) dma(1, 1, true);
        if (nst > 1) ST_WAIT_VM_LGKM0(kDma); else ST_WAIT_VM_LGKM0(0);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        rdB(Bc, 0);
        rdA(A[0], 0, 0);
        ST_TL(1);
        int nsafe = n / kPfBK2 - ks0;   // stages of this split that lie below row n as a whole
        nsafe = nsafe < nst ? nsafe : nst;
        int base = 0;
        for (; base + 5 <= nsafe; base += 3) {
            stage(0, base, false);
            stage(1, base + 1, false);
            stage(2, base + 2, false);
        }
        for (; base < nst; base += 3) {
            stage(0, base, true);
            if (base + 1 < nst) stage(1, base + 1, true);
            if (base + 2 < nst) stage(2, base + 2, true);
        }
    }

    ST_TL(2);
    // the pair's sums (see prefill_gateup_wide_kernel): kh = 0 finishes the first 64 rows of the tile, kh = 1 the last
    f32x4_t *red = reinterpret_cast<f32x4_t *>(lds);
    f32x4_t f[4][4];
    {
        f32x4_t *mine = red + (size_t)wave * 16 * 64 + lane;
        auto hand = [&](int h) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    mine[(i * 4 + j) * 64] = acc[4 * h + i][j];
                    f[i][j] = acc[4 * (1 - h) + i][j];
                }
        };
        if (kh == 0) hand(1); else hand(0);
    }
    __syncthreads();
    {
        const f32x4_t *other = red + (size_t)(wave ^ 4) * 16 * 64 + lane;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) f[i][j] += other[(i * 4 + j) * 64];
    }
    __syncthreads();

    ST_TL(3);
    static_assert(8 * 64 * kPfStgF * 4 <= (int)sizeof(lds), "staging tiles exceed the stage buffers");
    float *stg = reinterpret_cast<float *>(lds) + (size_t)wave * 64 * kPfStgF;
    pf_store_out<T>(f, stg, lane, m0 + 128 * wm + 64 * kh, c0 + 64 * wn, M, H, Out,
                    split_k == 1 ? nullptr : partial + (size_t)z * M * H);
    ST_TL(4);
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
    // (T is a 16-bit type here; M * H is a multiple of 4 and `out` a tensor's base, so the four results are one 8-byte store)
    const uint32_t lo = (uint32_t)from_float<T>(s.x).bits | ((uint32_t)from_float<T>(s.y).bits << 16);
    const uint32_t hi = (uint32_t)from_float<T>(s.z).bits | ((uint32_t)from_float<T>(s.w).bits << 16);
    if ((reinterpret_cast<uintptr_t>(out) & 7) == 0) {
        *reinterpret_cast<uint2 *>(out + i4) = make_uint2(lo, hi);
    } else {
        T *o = out + i4;
        o[0] = from_float<T>(s.x); o[1] = from_float<T>(s.y); o[2] = from_float<T>(s.z); o[3] = from_float<T>(s.w);
    }
}

int prefill_split_k(int M, int H, int n)
{
    // Two blocks fit a CU, so the blocks run in rounds of 2 x CUs; a split costs its K stages plus about four
    // stages of prologue and epilogue per round.  Take the split with the least rounds x stages.
    const int tiles = ((M + kPfBM - 1) / kPfBM) * ((H + kPfBN - 1) / kPfBN);
    const int slots = 2 * device_cu_count();
    const int nk = (n + kPfBK - 1) / kPfBK * (kPfBK / kPfBK2);   // K stages of 64
    int best = 1;
    long best_cost = -1;
    for (int s = 1; s <= 16; ++s) {
        if (s > 1 && s > nk / 8) break;   // keep at least 8 K stages per split
        const long rounds = ((long)tiles * s + slots - 1) / slots;
        const long cost = rounds * ((nk + s - 1) / s + 4);
        if (best_cost < 0 || cost < best_cost) { best = s; best_cost = cost; }
    }
    return best;
}

// The wide down kernel: 256-row tiles, one block per CU.  Taken when the row tiles waste at most a fifth of
// their rows; the K split then fills the CUs (at least 8 stages of 64 per split, at most 16 splits).
static bool prefill_down_is_wide(int M, int H, int n, long ldh)
{
    const int mt = (M + kPwBM - 1) / kPwBM;
    // (the wide kernels address their operands with 32-bit byte offsets: Hh and the rows of Wd have to stay below 4 GiB)
    return M > 128 && (mt * kPwBM - M) * 5 <= mt * kPwBM && H % kPfBN == 0 && n >= 512 &&
           (int64_t)M * ldh * 2 < ((int64_t)1 << 32) && (int64_t)n * H * 2 < ((int64_t)1 << 32);
}

static int prefill_split_k_wide(int M, int H, int n)
{
    const int tiles = ((M + kPwBM - 1) / kPwBM) * ((H + kPfBN - 1) / kPfBN);
    const int nk = (n + kPfBK - 1) / kPfBK * (kPfBK / kPfBK2);
    int s = device_cu_count() / tiles;
    if (s > nk / 8) s = nk / 8;
    if (s > 16) s = 16;
    return s < 1 ? 1 : s;
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
    // The intermediate Hh normally sits in the workspace, padded with zero columns to a multiple of 128.  When the
    // caller's combined buffer can take that padding (16-byte aligned rows with room up to the padded width) the
    // gate/up kernel writes there only and the down kernel reads it back from there: one store of M x n less.
    const long ldw = (long)prefill_ldh(n);
    const bool alias = comb && ldc % 8 == 0 && ldc >= ldw && (reinterpret_cast<uintptr_t>(comb) & 15) == 0;
    const long ldh = alias ? ldc : ldw;
    T *Hh = alias ? static_cast<T *>(comb) : static_cast<T *>(workspace);
    if (alias) comb = nullptr;
    const int64_t hh_bytes = (((int64_t)M * ldw * 2) + 255) & ~(int64_t)255;
    float *partial = reinterpret_cast<float *>(static_cast<unsigned char *>(workspace) + hh_bytes);
    const bool wide_down = prefill_down_is_wide(M, H, n, ldh);
    const int split_k = wide_down ? prefill_split_k_wide(M, H, n) : prefill_split_k(M, H, n);
    {
        ProfScope ps(ST_K_MLP_PREFILL_GATEUP, stream);
        const int cus = device_cu_count();
        const int jt64 = (int)(ldw / 64), mt128 = (M + 127) / 128;
        // 256-row blocks with 64 + 64 weight rows (one per CU, 25 % less operand traffic; the wide kernel) once
        // 128-row tiles outnumber the CUs.  Below that the K loop of a block, not the chip, is what takes the time: two thread
        // groups per tile with half of K each, on 128 x (64 + 64) tiles while those number more than half the
        // CUs and on 128 x (32 + 32) tiles (twice the blocks) when there are fewer -- four groups with a quarter
        // of K each on 64 x (32 + 32) tiles while those fit one per CU.  What is left (one row tile and more
        // than 16384 active rows) takes 128 x (32 + 32) tiles without K groups.
        // (32-bit byte offsets into x and the weight rows in the wide kernel)
        const bool big = M > 128 && jt64 * mt128 > cus && (int64_t)(M > n ? M : n) * H * 2 < ((int64_t)1 << 32);
        const bool halves = !big && 2 * jt64 * mt128 <= cus;
        // 64-row tiles: four K groups fit the LDS
        const bool quarters = !big && H % 256 == 0 && 2 * jt64 * ((M + 63) / 64) <= cus;
        const bool wide_halves = !big && !halves && jt64 * mt128 <= cus;   // K groups on 64 + 64 rows: one block per CU
        const int jt = big || (wide_halves && !quarters) ? jt64 : 2 * jt64;
        const int mt = big ? (M + 255) / 256 : quarters ? (M + 63) / 64 : mt128;
        const int grid = (jt * mt + kXcds - 1) / kXcds * kXcds;
        auto go = [&](auto kern, int threads) -> int {
            ST_LAUNCH(ps, kern, dim3(grid), dim3(threads), 0, stream, static_cast<const T *>(x),
                      static_cast<const T *>(gate), static_cast<const T *>(up), n_dev, M, H, n, jt, mt, Hh, ldh,
                      static_cast<T *>(comb), ldc, act);
            return ST_OK;
        };
        int rc;
        if (big) rc = has_gate ? go(prefill_gateup_wide_kernel<T, true>, kPwThreads) : go(prefill_gateup_wide_kernel<T, false>, kPwThreads);
        else if (quarters) rc = has_gate ? go(prefill_gateup_kernel<T, true, 64, 2, 4, 1>, 512) : go(prefill_gateup_kernel<T, false, 64, 2, 4, 1>, 512);
        else if (halves) rc = has_gate ? go(prefill_gateup_kernel<T, true, 128, 2, 2, 1>, 512) : go(prefill_gateup_kernel<T, false, 128, 2, 2, 1>, 512);
        else if (wide_halves) rc = has_gate ? go(prefill_gateup_kernel<T, true, 128, 2, 2, 2>, 512) : go(prefill_gateup_kernel<T, false, 128, 2, 2, 2>, 512);
        else rc = has_gate ? go(prefill_gateup_kernel<T, true, 128, 2, 1, 1>, 256) : go(prefill_gateup_kernel<T, false, 128, 2, 1, 1>, 256);
        if (rc != ST_OK) return rc;
    }
    ST_HIP(hipGetLastError());
    {
        ProfScope ps(ST_K_MLP_PREFILL_DOWN, stream);
        if (wide_down) {
            const int ct = (H + kPfBN - 1) / kPfBN, mt = (M + kPwBM - 1) / kPwBM;
            const int grid = (ct * mt * split_k + kXcds - 1) / kXcds * kXcds;
            ST_LAUNCH(ps, prefill_down_wide_kernel<T>, dim3(grid), dim3(kPwThreads), 0, stream, Hh,
                      static_cast<const T *>(down), n_dev, ldh, M, H, n, split_k, ct, mt, static_cast<T *>(out), partial);
        } else {
            const int ct = (H + kPfBN - 1) / kPfBN, mt = (M + kPfBM - 1) / kPfBM;
            const int grid = (ct * mt * split_k + kXcds - 1) / kXcds * kXcds;
            ST_LAUNCH(ps, prefill_down_kernel<T>, dim3(grid), dim3(kPfThreads), 0, stream, Hh,
                      static_cast<const T *>(down), n_dev, ldh, M, H, n, split_k, ct, mt, static_cast<T *>(out), partial);
        }
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
