// Row-wise selection on a score matrix [B, I] -> union-over-rows byte mask.
//
//   top-k        per row the k largest scores are active (equal scores: lower index first)
//                SkipDecoderLayer._compute_binary_mask, src/modeling_skip.py:208-211
//   statistical  per row: score > mean + std_pop * z, population std, strict >
//                _gaussian_topk, src/modeling_skip.py:197-202
//   union        any(dim=0), src/modeling_skip.py:214
//   sketch       approx_topk_threshold, sparse_transformers/csrc/approx_topk.h:10-88
//
// One block per row.  The row is read from HBM once; every thread keeps its scores in registers (rows of up
// to 16384 scores) as order-preserving 32-bit keys.  The k-th largest key is found exactly by a radix select
// (8-bit digits, most significant first, one LDS histogram per digit; once at most 64 keys share the
// prefix one wave ranks them directly), so nothing is sorted.  With several rows every block leaves its row mask
// in the workspace and the block that finishes last ORs them together; which block that is does not
// change the result.
#include "st_common.h"

namespace st {

constexpr int kSelThreads = 1024;
constexpr int kSelWaves = kSelThreads / kWave;
constexpr int kSelMaxLdsKeys = 36 * 1024;  // 144 KB of keys next to the small shared struct

// float -> unsigned key with the same order (-0 and +0 share one key, as they compare equal)
__device__ __forceinline__ uint32_t order_key(float v)
{
    uint32_t u = __float_as_uint(v);
    if (u == 0x80000000u) u = 0u;
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k)
{
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}

constexpr int kHistCopies = 8;  // a digit's counter exists once per lane % 8: equal digits in a wave spread over banks

struct SelShared {
    uint32_t hist[256 * kHistCopies];
    uint32_t hsum[256];
    uint32_t cand[kWave];
    uint32_t digit, rem, cnt, ncand;
    int wave_tot[kSelWaves];
    double wave_sum[kSelWaves];
    int last;
};

// k-th largest (1 <= k <= number of keys) of the block's keys.  `sweep(fn)` calls fn(key) for every key
// this thread owns.  Returns the key; `rem` = how many of the keys equal to it belong to the k largest
// (1..cnt), `cnt` = how many keys equal it.  Every thread of the block calls.
template <typename Sweep>
__device__ __forceinline__ uint32_t radix_select_desc(Sweep sweep, uint32_t k, SelShared &sh, int tid,
                                                      uint32_t &rem_out, uint32_t &cnt_out)
{
    const int copy = tid & (kHistCopies - 1);
    uint32_t prefix = 0u, pmask = 0u, rem = k, cnt = 0u;
    for (int shift = 24; shift >= 0; shift -= 8) {
        sh.hist[tid] = 0u;
        sh.hist[tid + kSelThreads] = 0u;
        static_assert(256 * kHistCopies == 2 * kSelThreads, "two counters per thread");
        __syncthreads();
        sweep([&](uint32_t kv) {
            if ((kv & pmask) == prefix) atomicAdd(&sh.hist[((kv >> shift) & 255u) * kHistCopies + copy], 1u);
        });
        __syncthreads();
        if (tid < 256) {
            uint32_t t = 0u;
#pragma unroll
            for (int c = 0; c < kHistCopies; ++c) t += sh.hist[tid * kHistCopies + c];
            sh.hsum[tid] = t;
        }
        __syncthreads();
        if (tid < kWave) {  // lane l owns digits 4l .. 4l+3; find the digit that holds the rem-th largest
            uint32_t h[4], local = 0u;
#pragma unroll
            for (int j = 0; j < 4; ++j) { h[j] = sh.hsum[4 * tid + j]; local += h[j]; }
            uint32_t incl = local;  // sum over lanes >= this one
#pragma unroll
            for (int off = 1; off < kWave; off <<= 1) {
                const uint32_t t = __shfl_down(incl, off, kWave);
                if (tid + off < kWave) incl += t;
            }
            uint32_t above = incl - local;  // keys whose digit is larger than 4l+3
#pragma unroll
            for (int j = 3; j >= 0; --j) {
                if (above < rem && rem <= above + h[j]) {
                    sh.digit = (uint32_t)(4 * tid + j);
                    sh.rem = rem - above;
                    sh.cnt = h[j];
                }
                above += h[j];
            }
        }
        __syncthreads();
        prefix |= sh.digit << shift;
        pmask |= 255u << shift;
        rem = sh.rem;
        cnt = sh.cnt;
        if (shift > 0 && cnt <= (uint32_t)kWave) {
            // Few keys are left under this prefix: list them and let one wave rank them directly instead
            // of spending a full pass on each remaining digit.  (cnt is uniform over the block.)
            if (tid == 0) sh.ncand = 0u;
            __syncthreads();
            sweep([&](uint32_t kv) {
                if ((kv & pmask) == prefix) sh.cand[atomicAdd(&sh.ncand, 1u)] = kv;
            });
            __syncthreads();
            if (tid < kWave) {
                const uint32_t mine = (uint32_t)tid < cnt ? sh.cand[tid] : 0u;
                uint32_t greater = 0u, equal = 0u;
                for (uint32_t j = 0; j < cnt; ++j) {
                    const uint32_t c = sh.cand[j];
                    greater += c > mine;
                    equal += c == mine;
                }
                if ((uint32_t)tid < cnt && greater < rem && rem <= greater + equal) {  // lanes that agree write the same
                    sh.digit = mine;
                    sh.rem = rem - greater;
                    sh.cnt = equal;
                }
            }
            __syncthreads();
            rem_out = sh.rem;
            cnt_out = sh.cnt;
            return sh.digit;
        }
    }
    rem_out = rem;
    cnt_out = cnt;
    return prefix;
}

__device__ __forceinline__ double block_sum(double v, SelShared &sh, int tid)
{
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
    __syncthreads();  // the previous reader of wave_sum is done
    if ((tid & (kWave - 1)) == 0) sh.wave_sum[tid >> 6] = v;
    __syncthreads();
    double s = 0.0;
#pragma unroll
    for (int w = 0; w < kSelWaves; ++w) s += sh.wave_sum[w];
    return s;
}

// Exclusive prefix of one int per thread, threads in order.
__device__ __forceinline__ int block_excl_count(int v, SelShared &sh, int tid)
{
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    int incl = v;
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const int t = __shfl_up(incl, off, kWave);
        if (lane >= off) incl += t;
    }
    if (lane == kWave - 1) sh.wave_tot[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += sh.wave_tot[w];
    return base + incl - v;
}

// KPT > 0: the row has at most KPT * 1024 scores and every thread keeps its KPT of them (index
// tid + u * 1024) in registers for all passes; a copy of the keys in LDS serves the one step that walks the
// row in index order.  KPT == 0: rows of any length, every pass reads the keys from LDS (`in_lds`) or the
// scores again from memory.
template <int KPT>
__global__ __launch_bounds__(kSelThreads) void mask_select_kernel(const float *__restrict__ scores,
                                                                  uint8_t *__restrict__ mask,
                                                                  uint8_t *__restrict__ rowmask,
                                                                  float *__restrict__ cutoff,
                                                                  unsigned int *__restrict__ ticket, int B, int I,
                                                                  int ldm, int method_word, long k_in, float z)
{
    // (pointers and sizes first: the first 14 dwords of the arguments are in scalar registers when the wave starts)
    const int method = method_word & 0xff, in_lds = (method_word >> 8) & 1;
    constexpr int NR = KPT > 0 ? KPT : 1;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ SelShared sh;
    uint32_t *keys = reinterpret_cast<uint32_t *>(smem);
    const int tid = threadIdx.x, b = blockIdx.x;
    const float *row = scores + (size_t)b * I;
    uint8_t *dst = B == 1 ? mask : rowmask + (size_t)b * ldm;

    float v[NR];
    if constexpr (KPT > 0) {  // all loads of the row are in flight together
#pragma unroll
        for (int u = 0; u < KPT; ++u) {
            const int i = tid + u * kSelThreads;
            v[u] = row[i < I ? i : I - 1];
        }
    }
    // fn(index, score) for every score of this thread
    auto each = [&](auto &&fn) __attribute__((always_inline)) {
        if constexpr (KPT > 0) {
#pragma unroll
            for (int u = 0; u < KPT; ++u)
                if (tid + u * kSelThreads < I) fn(tid + u * kSelThreads, v[u]);
        } else {
            for (int i = tid; i < I; i += kSelThreads)
                fn(i, in_lds && method == ST_MASK_TOPK ? key_value(keys[i]) : row[i]);
        }
    };

    if (method == ST_MASK_TOPK) {
        const uint32_t k = k_in < 0 ? 0u : (k_in > I ? (uint32_t)I : (uint32_t)k_in);
        if (k == 0u || k == (uint32_t)I) {  // nothing / everything (uniform over the block)
            each([&](int i, float) { dst[i] = k ? 1 : 0; });
        } else {
            if (KPT > 0 || in_lds) {
                if constexpr (KPT > 0) each([&](int i, float f) { keys[i] = order_key(f); });
                else for (int i = tid; i < I; i += kSelThreads) keys[i] = order_key(row[i]);
            }
            auto sweep = [&](auto &&fn) __attribute__((always_inline)) {
                each([&](int, float f) { fn(order_key(f)); });
            };
            uint32_t rem, cnt;
            const uint32_t kth = radix_select_desc(sweep, k, sh, tid, rem, cnt);
            if (cutoff && tid == 0) cutoff[b] = key_value(kth);
            if (rem == cnt) {  // every score equal to the k-th belongs to the k largest
                each([&](int i, float f) { dst[i] = order_key(f) >= kth ? 1 : 0; });
            } else {
                // only the first `rem` of the equal scores, by index: threads take contiguous index ranges
                auto key = [&](int i) { return (KPT > 0 || in_lds) ? keys[i] : order_key(row[i]); };
                const int per = (I + kSelThreads - 1) / kSelThreads;
                const int i0 = tid * per < I ? tid * per : I, i1 = i0 + per < I ? i0 + per : I;
                int eq = 0;
                for (int i = i0; i < i1; ++i) eq += key(i) == kth;
                int seen = block_excl_count(eq, sh, tid);
                for (int i = i0; i < i1; ++i) {
                    const uint32_t kv = key(i);
                    bool on = kv > kth;
                    if (kv == kth) { on = (uint32_t)seen < rem; ++seen; }
                    dst[i] = on ? 1 : 0;
                }
            }
        }
    } else {
        double s = 0.0;
        each([&](int, float f) { s += (double)f; });
        const double mean = block_sum(s, sh, tid) / (double)I;
        double q = 0.0;
        each([&](int, float f) { const double d = (double)f - mean; q += d * d; });
        const double var = block_sum(q, sh, tid) / (double)I;
        const float cut = (float)mean + (float)sqrt(var) * z;
        if (cutoff && tid == 0) cutoff[b] = cut;
        each([&](int i, float f) { dst[i] = f > cut ? 1 : 0; });
    }
    if (B == 1) return;

    // ---- union over rows by the block that finishes last
    for (int i = I + tid; i < ldm; i += kSelThreads) dst[i] = 0;  // padding of the row
    __syncthreads();
    if (tid == 0) {  // one release / acquire per block: the barriers on either side extend it to every thread
        __threadfence();
        sh.last = atomicAdd(ticket, 1u) == (unsigned int)(B - 1);
        __threadfence();
    }
    __syncthreads();
    if (!sh.last) return;
    const bool aligned = (reinterpret_cast<uintptr_t>(mask) & 15) == 0;
    for (int c = tid; c * 16 < I; c += kSelThreads) {
        uint4 acc = make_uint4(0u, 0u, 0u, 0u);
        for (int r0 = 0; r0 < B; r0 += 8) {
            uint4 w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) w[u] = ld16(rowmask + (size_t)(r0 + u < B ? r0 + u : B - 1) * ldm + c * 16);
#pragma unroll
            for (int u = 0; u < 8; ++u) { acc.x |= w[u].x; acc.y |= w[u].y; acc.z |= w[u].z; acc.w |= w[u].w; }
        }
        if (aligned && c * 16 + 16 <= I) {
            st16(mask + c * 16, acc);
        } else {
            const uint32_t w[4] = {acc.x, acc.y, acc.z, acc.w};
            for (int e = 0; e < 16 && c * 16 + e < I; ++e) mask[c * 16 + e] = (uint8_t)((w[e >> 2] >> (8 * (e & 3))) & 0xffu);
        }
    }
    if (tid == 0) *ticket = 0u;  // ready for the next call
}

// approx_topk_threshold: four max-sketches of width W per row; cell (s, p) holds the largest score of the
// features f with (s*F + f) % W == p (the reference hashes with std::hash<int64_t>, the identity).  The
// threshold is the sketch_k-th largest cell times 0.9, sketch_k = max(1, k * cells / F).
__global__ __launch_bounds__(kSelThreads) void approx_topk_kernel(const float *__restrict__ scores, int F, long k,
                                                                 int W, float *__restrict__ threshold)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ SelShared sh;
    uint32_t *cell = reinterpret_cast<uint32_t *>(smem);  // [4][W], W <= 1024
    const int tid = threadIdx.x, b = blockIdx.x;
    const float *row = scores + (size_t)b * F;
    const uint32_t kNegInf = order_key(-__builtin_inff());
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (tid + u * kSelThreads < 4 * W) cell[tid + u * kSelThreads] = kNegInf;
    __syncthreads();
    // position of feature f in sketch s: (s*F + f) % W = (off[s] + f % W) % W, with f % W advanced by
    // 1024 % W per iteration instead of a division per feature
    int off[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) off[s] = (int)(((long)s * F) % W);
    const int step = kSelThreads % W;
    int p = tid % W;
    for (int f0 = tid; f0 < F; f0 += 8 * kSelThreads) {
        float fv[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int f = f0 + u * kSelThreads;
            fv[u] = row[f < F ? f : F - 1];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (f0 + u * kSelThreads < F) {
                const uint32_t kv = order_key(fv[u]);
#pragma unroll
                for (int s = 0; s < 4; ++s) {
                    int q = p + off[s];
                    if (q >= W) q -= W;
                    atomicMax(&cell[s * W + q], kv);
                }
            }
            p += step;
            if (p >= W) p -= W;
        }
    }
    __syncthreads();
    uint32_t kr[4];
    int filled = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = tid + u * kSelThreads;
        kr[u] = i < 4 * W ? cell[i] : kNegInf;
        filled += kr[u] != kNegInf;
    }
    const long cells = (long)(block_sum((double)filled, sh, tid) + 0.5);
    if (cells == 0) {
        if (tid == 0) threshold[b] = 0.f;
        return;
    }
    long sk = k * cells / F;
    if (sk < 1) sk = 1;
    if (sk > cells) sk = cells;
    uint32_t rem, cnt;
    auto sweep = [&](auto &&fn) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (tid + u * kSelThreads < 4 * W) fn(kr[u]);
    };
    const uint32_t kth = radix_select_desc(sweep, (uint32_t)sk, sh, tid, rem, cnt);
    if (tid == 0) threshold[b] = key_value(kth) * 0.9f;
}

// The same for double scores (the reference dispatches on every floating type, approx_topk.h:33).  Cells are 64-bit
// order-preserving keys; the k-th largest is found by the 32-bit radix select twice: on the upper halves, then --
// among the keys that share the winning upper half -- on the lower halves.
__device__ __forceinline__ unsigned long long order_key64(double v)
{
    unsigned long long u = (unsigned long long)__double_as_longlong(v);
    if (u == 0x8000000000000000ull) u = 0ull;
    return (u >> 63) ? ~u : (u | 0x8000000000000000ull);
}
__device__ __forceinline__ double key_value64(unsigned long long k)
{
    return __longlong_as_double((long long)((k >> 63) ? (k & 0x7fffffffffffffffull) : ~k));
}

__global__ __launch_bounds__(kSelThreads) void approx_topk_f64_kernel(const double *__restrict__ scores, int F, long k,
                                                                     int W, double *__restrict__ threshold)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ SelShared sh;
    unsigned long long *cell = reinterpret_cast<unsigned long long *>(smem);  // [4][W], W <= 1024
    const int tid = threadIdx.x, b = blockIdx.x;
    const double *row = scores + (size_t)b * F;
    const unsigned long long kNegInf = order_key64(-__builtin_inf());
#pragma unroll
    for (int u = 0; u < 4; ++u)
        if (tid + u * kSelThreads < 4 * W) cell[tid + u * kSelThreads] = kNegInf;
    __syncthreads();
    for (int f = tid; f < F; f += kSelThreads) {
        const unsigned long long kv = order_key64(row[f]);
#pragma unroll
        for (int s = 0; s < 4; ++s) atomicMax(&cell[s * W + (int)(((long)s * F + f) % W)], kv);
    }
    __syncthreads();
    unsigned long long kr[4];
    int filled = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int i = tid + u * kSelThreads;
        kr[u] = i < 4 * W ? cell[i] : kNegInf;
        filled += kr[u] != kNegInf;
    }
    const long cells = (long)(block_sum((double)filled, sh, tid) + 0.5);
    if (cells == 0) {
        if (tid == 0) threshold[b] = 0.0;
        return;
    }
    long sk = k * cells / F;
    if (sk < 1) sk = 1;
    if (sk > cells) sk = cells;
    // (empty cells hold the key of -inf, the smallest there is: they never reach the sk <= cells largest)
    uint32_t rem, cnt;
    auto sweep_hi = [&](auto &&fn) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (tid + u * kSelThreads < 4 * W) fn((uint32_t)(kr[u] >> 32));
    };
    const uint32_t hi = radix_select_desc(sweep_hi, (uint32_t)sk, sh, tid, rem, cnt);
    const uint32_t want = rem;   // the rem-th largest lower half among the keys whose upper half is `hi`
    __syncthreads();
    auto sweep_lo = [&](auto &&fn) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (tid + u * kSelThreads < 4 * W && (uint32_t)(kr[u] >> 32) == hi) fn((uint32_t)kr[u]);
    };
    const uint32_t lo = radix_select_desc(sweep_lo, want, sh, tid, rem, cnt);
    if (tid == 0) threshold[b] = key_value64(((unsigned long long)hi << 32) | lo) * 0.9;
}

}  // namespace st

extern "C" int64_t st_mask_select_workspace_bytes(int64_t B, int64_t I)
{
    if (B < 1 || I < 1) return 0;
    return 16 + B * ((I + 15) / 16 * 16);
}

extern "C" int st_mask_select(const float *scores, int64_t B, int64_t I, int method, int64_t k, float z,
                              uint8_t *mask, float *cutoff, void *workspace, int64_t workspace_bytes, void *stream)
{
    using namespace st;
    ST_REQUIRE(scores && mask, "st_mask_select: null pointer");
    ST_REQUIRE(method == ST_MASK_TOPK || method == ST_MASK_STATISTICAL, "st_mask_select: unknown method %d", method);
    ST_REQUIRE(B >= 1 && B <= 4096, "st_mask_select: B=%lld out of range [1,4096]", (long long)B);
    ST_REQUIRE(I >= 1 && I <= (1 << 24), "st_mask_select: I=%lld out of range", (long long)I);
    const int ldm = (int)((I + 15) / 16 * 16);
    unsigned int *ticket = nullptr;
    uint8_t *rowmask = nullptr;
    if (B > 1) {
        ST_REQUIRE(workspace && workspace_bytes >= st_mask_select_workspace_bytes(B, I),
                   "st_mask_select: workspace of %lld bytes needed for B=%lld, I=%lld",
                   (long long)st_mask_select_workspace_bytes(B, I), (long long)B, (long long)I);
        ST_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 15) == 0, "st_mask_select: workspace must be 16-byte aligned");
        ticket = static_cast<unsigned int *>(workspace);
        rowmask = static_cast<uint8_t *>(workspace) + 16;
    }
    hipStream_t s = static_cast<hipStream_t>(stream);
    {
        const int rc = allow_dynamic_lds(reinterpret_cast<const void *>(mask_select_kernel<0>), kSelMaxLdsKeys * 4);
        if (rc != ST_OK) return rc;
    }
    ProfScope ps(ST_K_MASK_SELECT, s);
    const dim3 grid((unsigned)B), block(kSelThreads);
#define ST_SELECT_ARGS(in_lds) scores, mask, rowmask, cutoff, ticket, (int)B, (int)I, ldm, method | ((in_lds) << 8), (long)k, z
    if (I <= 8 * kSelThreads)
        ST_LAUNCH(ps, (mask_select_kernel<8>), grid, block, (size_t)I * 4, s, ST_SELECT_ARGS(1));
    else if (I <= 16 * kSelThreads)
        ST_LAUNCH(ps, (mask_select_kernel<16>), grid, block, (size_t)I * 4, s, ST_SELECT_ARGS(1));
    else if (I <= kSelMaxLdsKeys)
        ST_LAUNCH(ps, (mask_select_kernel<0>), grid, block, (size_t)I * 4, s, ST_SELECT_ARGS(1));
    else
        ST_LAUNCH(ps, (mask_select_kernel<0>), grid, block, 0, s, ST_SELECT_ARGS(0));
#undef ST_SELECT_ARGS
    ST_HIP(hipGetLastError());
    return ST_OK;
}

extern "C" int st_approx_topk_threshold(const float *scores, int64_t B, int64_t F, int64_t k, float *threshold,
                                        void *stream)
{
    using namespace st;
    ST_REQUIRE(scores && threshold, "st_approx_topk_threshold: null pointer");
    ST_REQUIRE(B >= 1 && B <= 65535, "st_approx_topk_threshold: B=%lld out of range", (long long)B);
    ST_REQUIRE(F >= 4 && F <= (1 << 24), "st_approx_topk_threshold: feature size %lld out of range [4, 2^24]",
               (long long)F);
    ST_REQUIRE(k > 0, "st_approx_topk_threshold: k must be positive");
    ST_REQUIRE(k <= F, "st_approx_topk_threshold: k cannot be larger than feature size");
    const int W = (int)(F / 4 < 1024 ? F / 4 : 1024);
    hipStream_t s = static_cast<hipStream_t>(stream);
    ProfScope ps(ST_K_MASK_SELECT, s);
    ST_LAUNCH(ps, approx_topk_kernel, dim3((unsigned)B), dim3(kSelThreads), (size_t)4 * W * 4, s, scores, (int)F, (long)k,
              W, threshold);
    ST_HIP(hipGetLastError());
    return ST_OK;
}

extern "C" int st_approx_topk_threshold_f64(const double *scores, int64_t B, int64_t F, int64_t k, double *threshold,
                                            void *stream)
{
    using namespace st;
    ST_REQUIRE(scores && threshold, "st_approx_topk_threshold_f64: null pointer");
    ST_REQUIRE(B >= 1 && B <= 65535, "st_approx_topk_threshold_f64: B=%lld out of range", (long long)B);
    ST_REQUIRE(F >= 4 && F <= (1 << 24), "st_approx_topk_threshold_f64: feature size %lld out of range [4, 2^24]",
               (long long)F);
    ST_REQUIRE(k > 0, "st_approx_topk_threshold_f64: k must be positive");
    ST_REQUIRE(k <= F, "st_approx_topk_threshold_f64: k cannot be larger than feature size");
    const int W = (int)(F / 4 < 1024 ? F / 4 : 1024);
    hipStream_t s = static_cast<hipStream_t>(stream);
    ProfScope ps(ST_K_MASK_SELECT, s);
    ST_LAUNCH(ps, approx_topk_f64_kernel, dim3((unsigned)B), dim3(kSelThreads), (size_t)4 * W * 8, s, scores, (int)F,
              (long)k, W, threshold);
    ST_HIP(hipGetLastError());
    return ST_OK;
}
