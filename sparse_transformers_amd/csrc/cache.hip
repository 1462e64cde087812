// Differential weight cache resident in HBM.
//
// update = ONE kernel.  Every block (1024 threads) first replays the
// bookkeeping of WeightCache::update_active_weights
// (sparse_transformers/csrc/weight_cache.h:229-359) redundantly in its own LDS
// (integer work only, identical in every block):
//   diff      ascending added / removed lists     (weight_cache.h:84-110)
//   phase 1   i-th removed position <- i-th added  (:248-277)   parallel
//   phase 2   surplus additions appended           (:280-307)   parallel
//   phase 3   surplus removals, swap-with-last     (:310-353)   one lane,
//             because each step depends on the list the previous one left
// and then copies its share of the changed rows with 16-byte loads/stores.
// The plan only decides WHICH index ends up at WHICH position.  Because every
// active row is a bit-copy of a pool row, the data movement never has to
// follow the sequential order: each position whose index changed is rewritten
// straight from the pool (no reads of the active buffers, hence no hazards
// between copies).
//
// The bookkeeping (index list, remembered mask, count) is double-buffered:
// blocks read buffer `epoch`, one block writes buffer `epoch ^ 1`, and the
// block that arrives last (a ticket counter packed with the epoch in one word)
// flips the epoch.  Nothing ever waits: a block that starts late still reads
// the old buffer, because nobody writes it during this launch.
#include "st_common.h"

#include <cstdlib>
#include <new>

namespace st {

constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / kWave;
constexpr uint16_t kNone = 0xffffu;
// LDS per intermediate element: pos(2) + idx(2) + added/removed lists(2) + flags(1) + dirty(1/8)
constexpr int64_t kPlanMaxI = 22000;

__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v, int lane)
{
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t o = __shfl_up(v, off, kWave);
        if (lane >= off) v += o;
    }
    return v;
}

// Exclusive scan of one uint32 per thread over the block; *total receives the sum.
template <int WAVES>
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t *wave_tot, uint32_t *total)
{
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t incl = wave_incl_scan(v, lane);
    __syncthreads();  // protect wave_tot from the previous use
    if (lane == kWave - 1) wave_tot[wave] = incl;
    __syncthreads();
    uint32_t prefix = 0, tot = 0;
    for (int w = 0; w < WAVES; ++w) {
        const uint32_t t = wave_tot[w];
        if (w < wave) prefix += t;
        tot += t;
    }
    *total = tot;
    return prefix + incl - v;
}

struct CopyPlan {
    const unsigned char *pool[3];
    unsigned char *active[3];
    int nmat;
    int row_bytes;
};

constexpr int kCopyUnroll = 4;  // rows a thread group keeps in flight

constexpr int kPlanMaxWords = 3;  // 8-element words per thread in the vector path: I <= 24576

__device__ __forceinline__ uint64_t nonzero_bytes(uint64_t x)
{
    x |= x >> 4; x |= x >> 2; x |= x >> 1;
    return x & 0x0101010101010101ull;
}

// VEC: I % 8 == 0 and the mask is 8-byte aligned, so masks are read as 8-byte
// words and indices as 16-byte vectors; both bookkeeping buffers are requested
// together with the ticket, so the kernel front costs one memory round trip.
template <bool VEC, int TPB>
__global__ __launch_bounds__(TPB) void cache_update_kernel(CopyPlan cp, const uint8_t *__restrict__ new_mask,
                                                                    uint8_t *__restrict__ cur_mask2,
                                                                    int32_t *__restrict__ indices2,
                                                                    int32_t *__restrict__ state, int I, int gs_log2)
{
    extern __shared__ __align__(16) unsigned char smem[];
    uint16_t *pos_l = reinterpret_cast<uint16_t *>(smem);  // index -> position
    uint16_t *idx_l = pos_l + I;                           // position -> index
    // added indices ascending from the front, removed indices ascending from the
    // back (k-th removed at lists[I-1-k]); the two never meet: na + nr <= I.
    // After the plan the same array holds the positions to rewrite.
    uint16_t *lists = idx_l + I;
    uint32_t *dirty = reinterpret_cast<uint32_t *>(lists + I + (I & 1));  // bit per position
    const int dirty_words = (I + 31) >> 5;
    uint8_t *flag_l = reinterpret_cast<uint8_t *>(dirty + ((dirty_words + 1) & ~1));  // bit0 new, bit1 old; 8-byte aligned
    __shared__ uint32_t wave_tot[(TPB / kWave)];
    __shared__ int n_new_s;
    __shared__ uint32_t ticket_s;

    const int tid = threadIdx.x;
    ST_TL(0);
    // Elements per thread (a contiguous range, so the diff lists come out ascending).
    const int E = VEC ? ((I + 8 * TPB - 1) / (8 * TPB)) * 8 : (I + TPB - 1) / TPB;
    const int e0 = tid * E < I ? tid * E : I, e1 = e0 + E < I ? e0 + E : I;

    uint64_t v_new[kPlanMaxWords], v_cur[2][kPlanMaxWords];
    int4 v_idx[2][kPlanMaxWords][2];
    int n_both[2];
    if constexpr (VEC) {
#pragma unroll
        for (int w = 0; w < kPlanMaxWords; ++w) {
            const int e = e0 + 8 * w;
            if (e < e1) {
                v_new[w] = *reinterpret_cast<const uint64_t *>(new_mask + e);
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    v_cur[b][w] = *reinterpret_cast<const uint64_t *>(cur_mask2 + (size_t)b * I + e);
                    v_idx[b][w][0] = *reinterpret_cast<const int4 *>(indices2 + (size_t)b * I + e);
                    v_idx[b][w][1] = *reinterpret_cast<const int4 *>(indices2 + (size_t)b * I + e + 4);
                }
            }
        }
        n_both[0] = state[ST_STATE_N_BUF0];
        n_both[1] = state[ST_STATE_N_BUF1];
    }
    // One atomic returns both the epoch (which buffer to read) and this block's ticket.
    if (tid == 0) ticket_s = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
    for (int w = tid; w < dirty_words; w += TPB) dirty[w] = 0u;
    __syncthreads();
    const uint32_t ticket = ticket_s;
    const int ep = (int)((ticket >> 16) & 1u);
    const bool last_arrival = (ticket & 0xffffu) == gridDim.x - 1;
    const bool writer = blockIdx.x == 0;

    int n;
    // VEC: new / current mask words as 0x01 bytes, kept in registers for the diff and for publishing
    uint64_t w_new[kPlanMaxWords], w_cur[kPlanMaxWords];
    if constexpr (VEC) {
        n = ep ? n_both[1] : n_both[0];
#pragma unroll
        for (int w = 0; w < kPlanMaxWords; ++w) {
            const int e = e0 + 8 * w;
            w_new[w] = w_cur[w] = 0;
            if (e < e1) {
                w_new[w] = nonzero_bytes(v_new[w]);
                w_cur[w] = nonzero_bytes(ep ? v_cur[1][w] : v_cur[0][w]);
                const int4 a = ep ? v_idx[1][w][0] : v_idx[0][w][0], b4 = ep ? v_idx[1][w][1] : v_idx[0][w][1];
                uint4 packed;
                packed.x = (uint32_t)(a.x & 0xffff) | ((uint32_t)a.y << 16);
                packed.y = (uint32_t)(a.z & 0xffff) | ((uint32_t)a.w << 16);
                packed.z = (uint32_t)(b4.x & 0xffff) | ((uint32_t)b4.y << 16);
                packed.w = (uint32_t)(b4.z & 0xffff) | ((uint32_t)b4.w << 16);
                *reinterpret_cast<uint4 *>(idx_l + e) = packed;
                *reinterpret_cast<uint4 *>(pos_l + e) = make_uint4(0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu);
            }
        }
    } else {
        const uint8_t *cur_mask = cur_mask2 + (size_t)ep * I;
        const int32_t *indices = indices2 + (size_t)ep * I;
        n = state[ST_STATE_N_BUF0 + ep];
        for (int i = tid; i < I; i += TPB) {
            pos_l[i] = kNone;
            flag_l[i] = (new_mask[i] ? 1 : 0) | (cur_mask[i] ? 2 : 0);
            idx_l[i] = (uint16_t)indices[i];
        }
    }
    ST_TL(1);
    __syncthreads();
    ST_TL(2);
    for (int p = tid; p < n; p += TPB) pos_l[idx_l[p]] = (uint16_t)p;

    // ---- diff: contiguous element range per thread keeps the lists ascending
    uint32_t cnt = 0;  // added in the low half, removed in the high half
    if constexpr (VEC) {
#pragma unroll
        for (int w = 0; w < kPlanMaxWords; ++w)
            cnt += (uint32_t)__popcll(w_new[w] & ~w_cur[w]) + ((uint32_t)__popcll(w_cur[w] & ~w_new[w]) << 16);
    } else {
        for (int i = e0; i < e1; ++i) {
            const uint8_t f = flag_l[i];
            cnt += (f == 1) ? 1u : 0u;
            cnt += (f == 2) ? 0x10000u : 0u;
        }
    }
    uint32_t total;
    const uint32_t off = block_excl_scan<TPB / kWave>(cnt, wave_tot, &total);  // contains __syncthreads
    ST_TL(3);
    const int na = (int)(total & 0xffffu), nr = (int)(total >> 16);
    if (na == 0 && nr == 0) {  // unchanged mask: nothing is touched (weight_cache.h:237-240)
        if (tid == 0) {
            if (last_arrival) atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)ep << 16);
            if (writer) {
                state[ST_STATE_N_CHANGED] = 0;
                state[ST_STATE_N_ADDED] = 0;
                state[ST_STATE_N_REMOVED] = 0;
            }
        }
        return;
    }
    {
        int oa = (int)(off & 0xffffu), orr = (int)(off >> 16);
        if constexpr (VEC) {
#pragma unroll
            for (int w = 0; w < kPlanMaxWords; ++w) {
                const int e = e0 + 8 * w;
                uint64_t a = w_new[w] & ~w_cur[w], r = w_cur[w] & ~w_new[w];   // one 0x01 byte per element, ascending
                while (a) {
                    lists[oa++] = (uint16_t)(e + ((__ffsll((long long)a) - 1) >> 3));
                    a &= a - 1;
                }
                while (r) {
                    lists[I - 1 - (orr++)] = (uint16_t)(e + ((__ffsll((long long)r) - 1) >> 3));
                    r &= r - 1;
                }
            }
        } else {
            for (int i = e0; i < e1; ++i) {
                const uint8_t f = flag_l[i];
                if (f == 1) lists[oa++] = (uint16_t)i;
                if (f == 2) lists[I - 1 - (orr++)] = (uint16_t)i;
            }
        }
    }
    __syncthreads();

    const int pairs = na < nr ? na : nr;
    // Without surplus removals (nr <= na) the rewritten positions are known as soon as phases 1 and 2
    // have run: they replace the added indices in `lists` in place and no compaction is needed.
    const bool fast = nr <= na;
    // ---- phase 1: paired replacement
    for (int i = tid; i < pairs; i += TPB) {
        const int e = lists[I - 1 - i];
        const uint16_t p = pos_l[e];
        if (p != kNone) {
            const int a = lists[i];
            idx_l[p] = (uint16_t)a;
            pos_l[a] = p;
            pos_l[e] = kNone;
            if (!fast) atomicOr(&dirty[p >> 5], 1u << (p & 31));
        }
        if (fast) lists[i] = p;
    }
    // ---- phase 2: append surplus additions
    for (int i = pairs + tid; i < na; i += TPB) {
        const int p = n + (i - pairs);
        if (p < I) {
            const int a = lists[i];
            idx_l[p] = (uint16_t)a;
            pos_l[a] = (uint16_t)p;
        }
        lists[i] = p < I ? (uint16_t)p : kNone;
    }
    __syncthreads();

    int n_new;
    uint32_t n_changed;
    if (fast) {
        n_new = n + (na - pairs);
        if (n_new > I) n_new = I;
        n_changed = (uint32_t)na;
        ST_TL(4);
    } else {
        // ---- phase 3: surplus removals, sequential by construction
        if (tid == 0) {
            int m = n;
            for (int k = pairs; k < nr; ++k) {
                const int e = lists[I - 1 - k];
                const uint16_t p = pos_l[e];
                if (p == kNone) continue;
                if (m <= 0) break;
                const int last = m - 1;
                if ((int)p != last) {
                    const uint16_t li = idx_l[last];
                    idx_l[p] = li;
                    pos_l[li] = p;
                    dirty[p >> 5] |= 1u << (p & 31);
                }
                --m;
                pos_l[e] = kNone;
            }
            n_new_s = m;
        }
        __syncthreads();
        ST_TL(4);
        n_new = n_new_s;

        // ---- compact the dirty positions below n_new into the copy list (in LDS, over the dead lists)
        uint32_t word = 0;
        if (tid < dirty_words) {
            word = dirty[tid];
            const int lo = tid << 5;
            if (lo >= n_new) word = 0;
            else if (lo + 32 > n_new) word &= (1u << (n_new - lo)) - 1u;
        }
        uint32_t coff = block_excl_scan<TPB / kWave>((uint32_t)__popc(word), wave_tot, &n_changed);  // barrier: lists are dead now
        while (word) {
            const int bit = __ffs(word) - 1;
            word &= word - 1;
            lists[coff++] = (uint16_t)((tid << 5) + bit);
        }
        __syncthreads();
    }

    ST_TL(5);
    // ---- copy this block's share of the changed rows: active[m][p] <- pool[m][index at p]
    {
        const int nmat = cp.nmat, row_bytes = cp.row_bytes, chunks = row_bytes >> 4;
        const int GS = 1 << gs_log2, ngrp = TPB >> gs_log2;
        const int grp = tid >> gs_log2, cc = tid & (GS - 1);
        // the publishing block takes no copies when there are others to do them
        const bool solo = gridDim.x == 1;
        const bool copies = solo || !writer;
        const int slots = (solo ? 1 : (int)gridDim.x - 1) * ngrp;
        const int slot = (solo ? 0 : (int)blockIdx.x - 1) * ngrp + grp;   // >= 0 whenever `copies`
        const int work = (int)n_changed * nmat;
        for (int w0 = copies ? slot : work; w0 < work; w0 += slots * kCopyUnroll) {
            for (int c = cc; c < chunks; c += GS) {
                uint4 v[kCopyUnroll];
                unsigned char *dst[kCopyUnroll];
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u) {
                    const int w = w0 + u * slots;
                    dst[u] = nullptr;
                    if (w < work) {
                        const int j = w / nmat, m = w - j * nmat;
                        const int p = lists[j];
                        if (p == kNone) continue;  // a removed index that was not in the cache: nothing to copy
                        const int idx = idx_l[p];
                        const unsigned char *pool = m == 0 ? cp.pool[0] : (m == 1 ? cp.pool[1] : cp.pool[2]);
                        unsigned char *act = m == 0 ? cp.active[0] : (m == 1 ? cp.active[1] : cp.active[2]);
                        v[u] = ld16(pool + (size_t)idx * row_bytes + ((size_t)c << 4));
                        dst[u] = act + (size_t)p * row_bytes + ((size_t)c << 4);
                    }
                }
#pragma unroll
                for (int u = 0; u < kCopyUnroll; ++u)
                    if (dst[u]) st16(dst[u], v[u]);
            }
        }
    }

    ST_TL(6);
    // ---- publish: one block writes the other bookkeeping buffer, the last arrival flips the epoch
    if (writer) {
        int32_t *idx_out = indices2 + (size_t)(ep ^ 1) * I;
        uint8_t *mask_out = cur_mask2 + (size_t)(ep ^ 1) * I;
        for (int p = tid; p < n_new; p += TPB) idx_out[p] = idx_l[p];
        // the reference stores the new mask only when the rebuild did not throw (n_new > 0)
        if constexpr (VEC) {
#pragma unroll
            for (int w = 0; w < kPlanMaxWords; ++w) {
                const int e = e0 + 8 * w;
                if (e < e1) *reinterpret_cast<uint64_t *>(mask_out + e) = n_new > 0 ? w_new[w] : w_cur[w];
            }
        } else {
            for (int i = tid; i < I; i += TPB) mask_out[i] = n_new > 0 ? (flag_l[i] & 1) : (flag_l[i] >> 1);
        }
        if (tid == 0) {
            state[ST_STATE_N_BUF0 + (ep ^ 1)] = n_new;
            state[ST_STATE_N_ACTIVE] = n_new;
            state[ST_STATE_N_CHANGED] = (int)n_changed;
            state[ST_STATE_N_ADDED] = na;
            state[ST_STATE_N_REMOVED] = nr;
            state[ST_STATE_SERIAL] += 1;
            state[ST_STATE_EPOCH] = ep ^ 1;
            if (n_new > 0) {
                state[ST_STATE_STATUS] = 0;
                state[ST_STATE_VALID] = 1;
            } else {
                state[ST_STATE_STATUS] = ST_ERR_NO_ACTIVE;
            }
        }
    }
    if (last_arrival && tid == 0)
        atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)(ep ^ 1) << 16);
    ST_TL(7);
}

// in [R,C] -> out [C,R], 64x64 tiles through LDS.
template <typename E>
__global__ __launch_bounds__(256) void transpose_kernel(const E *__restrict__ in, E *__restrict__ out, int R, int C)
{
    __shared__ E tile[64][65];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int c0 = blockIdx.x * 64, r0 = blockIdx.y * 64;
    for (int k = ty; k < 64; k += 4) {
        const int r = r0 + k, c = c0 + tx;
        if (r < R && c < C) tile[k][tx] = in[(size_t)r * C + c];
    }
    __syncthreads();
    for (int k = ty; k < 64; k += 4) {
        const int c = c0 + k, r = r0 + tx;
        if (r < R && c < C) out[(size_t)c * R + r] = tile[tx][k];
    }
}

__global__ void cache_reset_kernel(uint8_t *cur_mask2, int32_t *indices2, int32_t *state, int I)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < 2 * I) {
        cur_mask2[i] = 0;
        indices2[i] = -1;
    }
    if (i < ST_STATE_WORDS) state[i] = 0;
}

}  // namespace st

struct st_cache {
    st_cache_buffers b;
    int64_t I, H;
    int dtype, has_gate;
    int esz;
    int32_t *host_state;  // pinned
};

extern "C" int64_t st_cache_max_intermediate(void) { return st::kPlanMaxI; }

extern "C" st_cache *st_cache_create(const st_cache_buffers *bufs, int64_t I, int64_t H, int dtype, int has_gate)
{
    using namespace st;
    auto fail = [](const char *m) -> st_cache * { set_error("st_cache_create: %s", m); return nullptr; };
    if (!bufs) return fail("null buffers");
    if (dtype < ST_F32 || dtype > ST_BF16) return fail("unknown dtype");
    const int esz = dtype == ST_F32 ? 4 : 2;
    if (I < 1 || I > kPlanMaxI) return fail("intermediate size out of range (see st_cache_max_intermediate)");
    if (H < 1 || (H * esz) % 16 != 0) return fail("rows are not 16-byte multiples");
    if (!bufs->up_pool || !bufs->downT_pool || !bufs->up_active || !bufs->down_active || !bufs->indices ||
        !bufs->cur_mask || !bufs->state)
        return fail("null device buffer");
    if (has_gate && (!bufs->gate_pool || !bufs->gate_active)) return fail("has_gate set but gate buffers are null");
    const uintptr_t align = (uintptr_t)bufs->gate_pool | (uintptr_t)bufs->up_pool | (uintptr_t)bufs->downT_pool |
                            (uintptr_t)bufs->gate_active | (uintptr_t)bufs->up_active | (uintptr_t)bufs->down_active;
    if (align & 15) return fail("weight buffers must be 16-byte aligned");
    st_cache *c = new (std::nothrow) st_cache;
    if (!c) return fail("out of host memory");
    c->b = *bufs;
    c->I = I; c->H = H; c->dtype = dtype; c->has_gate = has_gate ? 1 : 0; c->esz = esz;
    c->host_state = nullptr;
    if (hipHostMalloc(reinterpret_cast<void **>(&c->host_state), ST_STATE_WORDS * sizeof(int32_t), hipHostMallocDefault) !=
        hipSuccess) {
        delete c;
        return fail("hipHostMalloc failed");
    }
    return c;
}

extern "C" void st_cache_destroy(st_cache *c)
{
    if (!c) return;
    if (c->host_state) (void)hipHostFree(c->host_state);
    delete c;
}

extern "C" int st_cache_load_weights(st_cache *c, const void *gate, const void *up, const void *down, void *stream)
{
    using namespace st;
    ST_REQUIRE(c && up && down, "st_cache_load_weights: null pointer");
    ST_REQUIRE(!c->has_gate || gate, "st_cache_load_weights: gated cache needs gate weights");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t bytes = (size_t)c->I * c->H * c->esz;
    ST_HIP(hipMemcpyAsync(c->b.up_pool, up, bytes, hipMemcpyDeviceToDevice, s));
    if (c->has_gate) ST_HIP(hipMemcpyAsync(c->b.gate_pool, gate, bytes, hipMemcpyDeviceToDevice, s));
    const dim3 grid((unsigned)((c->I + 63) / 64), (unsigned)((c->H + 63) / 64));
    if (c->esz == 4)
        hipLaunchKernelGGL(transpose_kernel<uint32_t>, grid, dim3(256), 0, s, static_cast<const uint32_t *>(down),
                           static_cast<uint32_t *>(c->b.downT_pool), (int)c->H, (int)c->I);
    else
        hipLaunchKernelGGL(transpose_kernel<uint16_t>, grid, dim3(256), 0, s, static_cast<const uint16_t *>(down),
                           static_cast<uint16_t *>(c->b.downT_pool), (int)c->H, (int)c->I);
    ST_HIP(hipGetLastError());
    hipLaunchKernelGGL(cache_reset_kernel, dim3((unsigned)((2 * c->I + 255) / 256)), dim3(256), 0, s, c->b.cur_mask,
                       c->b.indices, c->b.state, (int)c->I);
    ST_HIP(hipGetLastError());
    return ST_OK;
}

extern "C" int st_cache_update_async(st_cache *c, const uint8_t *mask, void *stream)
{
    using namespace st;
    ST_REQUIRE(c && mask, "st_cache_update_async: null pointer");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int I = (int)c->I;
    const size_t lds = (size_t)I * 6 + (I & 1) * 2 + (size_t)((((I + 31) >> 5) + 1) & ~1) * 4 + (size_t)I + 16;
    CopyPlan cp;
    cp.nmat = 0;
    if (c->has_gate) {
        cp.pool[cp.nmat] = static_cast<const unsigned char *>(c->b.gate_pool);
        cp.active[cp.nmat++] = static_cast<unsigned char *>(c->b.gate_active);
    }
    cp.pool[cp.nmat] = static_cast<const unsigned char *>(c->b.up_pool);
    cp.active[cp.nmat++] = static_cast<unsigned char *>(c->b.up_active);
    cp.pool[cp.nmat] = static_cast<const unsigned char *>(c->b.downT_pool);
    cp.active[cp.nmat++] = static_cast<unsigned char *>(c->b.down_active);
    for (int k = cp.nmat; k < 3; ++k) { cp.pool[k] = cp.pool[0]; cp.active[k] = cp.active[0]; }
    cp.row_bytes = (int)(c->H * c->esz);
    const int chunks = cp.row_bytes >> 4;
    static const int blocks = [] {
        const char *v = getenv("ST_CACHE_BLOCKS");
        const int b = v ? atoi(v) : 0;
        return b >= 1 && b <= 1024 ? b : 0;
    }();
    static const int want_tpb = [] {
        const char *v = getenv("ST_CACHE_TPB");
        return v ? atoi(v) : 0;
    }();
    const int grid = blocks ? blocks : device_cu_count() / 2;
    const bool aligned = (I % 8 == 0) && ((uintptr_t)mask % 8 == 0) && ((uintptr_t)c->b.cur_mask % 8 == 0) &&
                         ((uintptr_t)c->b.indices % 16 == 0);
    // 512-thread blocks (ST_CACHE_TPB=512) leave room on the CU for a kernel of another stream, but
    // measure slower on their own; they cover I <= 12288 in the vector path.
    const bool small = want_tpb == 512 && aligned && I <= 8 * 512 * kPlanMaxWords;
    const int tpb = small ? 512 : 1024;
    const bool vec = aligned && I <= 8 * tpb * kPlanMaxWords;
    int gs_log2 = 6;
    while ((1 << gs_log2) < chunks && (1 << gs_log2) < tpb) ++gs_log2;
    {
        ProfScope ps(ST_K_CACHE_UPDATE, s);
        auto launch = [&](auto kern) -> int {
            static bool attr_set = false;
            if (!attr_set) {
                ST_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256));
                attr_set = true;
            }
            hipLaunchKernelGGL(kern, dim3(grid), dim3(tpb), lds, s, cp, mask, c->b.cur_mask, c->b.indices, c->b.state,
                               I, gs_log2);
            return ST_OK;
        };
        int rc;
        if (small) rc = launch(cache_update_kernel<true, 512>);
        else if (vec) rc = launch(cache_update_kernel<true, 1024>);
        else rc = launch(cache_update_kernel<false, 1024>);
        if (rc != ST_OK) return rc;
    }
    ST_HIP(hipGetLastError());
    return ST_OK;
}

extern "C" int st_cache_sync_state(st_cache *c, int32_t *state_out, void *stream)
{
    using namespace st;
    ST_REQUIRE(c, "st_cache_sync_state: null handle");
    hipStream_t s = static_cast<hipStream_t>(stream);
    ST_HIP(hipMemcpyAsync(c->host_state, c->b.state, ST_STATE_WORDS * sizeof(int32_t), hipMemcpyDeviceToHost, s));
    ST_HIP(hipStreamSynchronize(s));
    if (state_out)
        for (int i = 0; i < ST_STATE_WORDS; ++i) state_out[i] = c->host_state[i];
    if (c->host_state[ST_STATE_STATUS] == ST_ERR_NO_ACTIVE) {
        set_error("No active weights");
        return ST_ERR_NO_ACTIVE;
    }
    return ST_OK;
}

extern "C" int st_cache_materialize_concat(st_cache *c, void *dst, int64_t n, void *stream)
{
    using namespace st;
    ST_REQUIRE(c && dst, "st_cache_materialize_concat: null pointer");
    ST_REQUIRE(n >= 1 && n <= c->I, "st_cache_materialize_concat: n=%lld out of range", (long long)n);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t blk = (size_t)n * c->H * c->esz;
    unsigned char *d = static_cast<unsigned char *>(dst);
    if (c->has_gate) {
        ST_HIP(hipMemcpyAsync(d, c->b.gate_active, blk, hipMemcpyDeviceToDevice, s));
        d += blk;
    }
    ST_HIP(hipMemcpyAsync(d, c->b.up_active, blk, hipMemcpyDeviceToDevice, s));
    return ST_OK;
}
