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

#include <atomic>

#include <cstdlib>
#include <new>
#include <type_traits>

namespace st {

constexpr int kPlanThreads = 1024;
constexpr int kPlanWaves = kPlanThreads / kWave;
constexpr uint16_t kNone = 0xffffu;
// LDS per intermediate element: pos(2) + idx(2) + added/removed lists(2) + flags(1) + dirty(1/8)
constexpr int64_t kPlanMaxI = 22000;

// Block barrier that orders LDS traffic only.  __syncthreads() also waits for every outstanding global
// load, which would serialise loads that are meant to stay in flight across the bookkeeping phases.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ uint32_t wave_incl_scan(uint32_t v, int lane)
{
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
        const uint32_t o = __shfl_up(v, off, kWave);
        if (lane >= off) v += o;
    }
    return v;
}

// The same with DPP row shifts (no LDS crossbar traffic): four steps scan each row of 16 lanes, the row totals
// travel through scalar registers.
template <int CTRL> __device__ __forceinline__ uint32_t dpp_shr_add(uint32_t v)
{
    return v + (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xf, 0xf, true);   // lanes shifted in from outside the row read 0
}
__device__ __forceinline__ uint32_t wave_incl_scan_dpp(uint32_t v, int lane)
{
    v = dpp_shr_add<0x111>(v);   // row_shr:1
    v = dpp_shr_add<0x112>(v);   // row_shr:2
    v = dpp_shr_add<0x114>(v);   // row_shr:4
    v = dpp_shr_add<0x118>(v);   // row_shr:8
    const uint32_t t0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 15), t1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 31),
                   t2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 47);
    const int row = lane >> 4;
    return v + (row >= 1 ? t0 : 0u) + (row >= 2 ? t1 : 0u) + (row >= 3 ? t2 : 0u);
}

// Exclusive scan of one uint32 per thread over WAVES waves; *total receives the sum.  `sync` is the
// barrier of exactly those waves.
template <int WAVES, typename S>
__device__ __forceinline__ uint32_t block_excl_scan(uint32_t v, uint32_t *wave_tot, uint32_t *total, int tid, S sync)
{
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const uint32_t incl = wave_incl_scan(v, lane);
    sync();  // protect wave_tot from the previous use
    if (lane == kWave - 1) wave_tot[wave] = incl;
    sync();
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

// The same matrices for the fused update + MLP kernel, by name (no arrays: nothing for the compiler to index).
// Without a gate the gate members repeat the up members and are not used.
struct FusedRows {
    const unsigned char *pool_g, *pool_u, *pool_d;
    unsigned char *act_g, *act_u, *act_d;
    int row_bytes, has_gate;
};

constexpr int kCopyUnroll = 4;  // rows a thread group keeps in flight

constexpr int kPlanMaxWords = 4;  // 8-element words per thread in the vector path: I <= 32 * threads

__device__ __forceinline__ uint64_t nonzero_bytes(uint64_t x)
{
    x |= x >> 4; x |= x >> 2; x |= x >> 1;
    return x & 0x0101010101010101ull;
}

// The plan as every block computes it, and the LDS arrays that hold it.
struct PlanView {
    uint16_t *pos_l;    // index -> position (kNone when absent)
    uint16_t *idx_l;    // position -> index, after the update
    uint16_t *lists;    // positions to rewrite: [0, n_changed)
    uint32_t *dirty;    // bit per position whose index changed (complete only with MARK, or on the slow path)
    int ep;             // bookkeeping buffer this launch read
    bool writer;        // this block publishes
    bool arriver;       // this thread issued the block's arrival
    uint32_t arrival;   // arriver only: ticket word before this block's arrival (requested, not yet looked at)
    int next_epoch;     // epoch the last arrival leaves behind
    bool changed;       // false: the mask equals the remembered one, nothing was touched
    int n_old, n_new, na, nr;
    uint32_t n_changed;
};

constexpr size_t plan_lds_bytes(int I)
{
    return (size_t)I * 6 + (size_t)(I & 1) * 2 + (size_t)((((I + 31) >> 5) + 1) & ~1) * 4 + (size_t)I + 16;
}

// Small block-wide scalars of the plan (static LDS, declared by the kernel so that waves which do not take
// part in the plan can read them).
struct PlanShared {
    uint32_t wave_tot[kPlanWaves];
    int n_new_s;   // count after the sequential removals (slow path)
};

// Replays the bookkeeping of one update in LDS and publishes it (block 0 writes the other bookkeeping
// buffer, the last block to arrive flips the epoch).  Called by all PT threads of the block (tid = 0..PT-1);
// contains block barriers.  VEC: I % 8 == 0 and the mask is
// 8-byte aligned, so masks are read as 8-byte words and indices as 16-byte vectors; both bookkeeping
// buffers are requested together with the ticket, so the front costs one memory round trip.  MARK: the
// dirty bitmap is kept on the fast path too.  `after_issue()` runs right after the front loads have
// been issued, `after_fill()` right after the first barrier (the front loads have arrived and been consumed).
// idx_cap: only that many positions of the index lists are fetched up front (the rest follows if the count
// turns out larger).
//
// Barrier sequence: 1 after the LDS fill; 2 in the diff scan;
// [unchanged mask: done]; 1 after the lists; 1 after phases 1 and 2; [surplus removals: 1 after phase 3,
// 2 in the compaction scan, 1 after the compaction].
template <bool VEC, int PT, bool MARK, typename F, typename F2>
__device__ __forceinline__ void cache_plan(PlanView &pv, unsigned char *smem, PlanShared *ps,
                                           const uint8_t *__restrict__ new_mask, uint8_t *__restrict__ cur_mask2,
                                           int32_t *__restrict__ indices2, int32_t *__restrict__ state, int I,
                                           const int idx_cap, const int tid, F after_issue, F2 after_fill)
{
    constexpr int TPB = PT;
    uint16_t *pos_l = reinterpret_cast<uint16_t *>(smem);  // index -> position
    uint16_t *idx_l = pos_l + I;                           // position -> index
    // added indices ascending from the front, removed indices ascending from the
    // back (k-th removed at lists[I-1-k]); the two never meet: na + nr <= I.
    // After the plan the same array holds the positions to rewrite.
    uint16_t *lists = idx_l + I;
    uint32_t *dirty = reinterpret_cast<uint32_t *>(lists + I + (I & 1));  // bit per position
    const int dirty_words = (I + 31) >> 5;
    uint8_t *flag_l = reinterpret_cast<uint8_t *>(dirty + ((dirty_words + 1) & ~1));  // bit0 new, bit1 old; 8-byte aligned
    uint32_t *wave_tot = ps->wave_tot;
    int &n_new_s = ps->n_new_s;
    auto sync = [&]() __attribute__((always_inline)) { lds_barrier(); };
    pv.pos_l = pos_l; pv.idx_l = idx_l; pv.lists = lists; pv.dirty = dirty;
    pv.arriver = tid == 0;

    ST_TL(0);
    // Elements per thread (a contiguous range, so the diff lists come out ascending).
    const int E = VEC ? ((I + 8 * TPB - 1) / (8 * TPB)) * 8 : (I + TPB - 1) / TPB;
    const int e0 = tid * E < I ? tid * E : I, e1 = e0 + E < I ? e0 + E : I;

    // The ticket word holds the epoch (bit 16: which buffer to read) and the arrivals so far.  Every thread
    // reads it with a plain load, together with the rest of the front; the epoch cannot flip before every
    // block has arrived, and a block arrives (one atomic, at the end of the plan) only after all its
    // threads have consumed this load, so they all see the same epoch.
    const uint32_t tword = __hip_atomic_load(reinterpret_cast<const uint32_t *>(&state[ST_STATE_TICKET]), __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);

    // (several small arrays rather than one big one: each has to stay below the size up to which the
    // compiler keeps a private array in registers)
    uint64_t v_new[kPlanMaxWords], v_cur0[kPlanMaxWords], v_cur1[kPlanMaxWords];
    int4 v_i0a[kPlanMaxWords], v_i0b[kPlanMaxWords], v_i1a[kPlanMaxWords], v_i1b[kPlanMaxWords];
    int n_both[2];
    if constexpr (VEC) {
#pragma unroll
        for (int w = 0; w < kPlanMaxWords; ++w) {
            const int e = e0 + 8 * w;
            if (e < e1) {
                v_new[w] = *reinterpret_cast<const uint64_t *>(new_mask + e);
                v_cur0[w] = *reinterpret_cast<const uint64_t *>(cur_mask2 + e);
                v_cur1[w] = *reinterpret_cast<const uint64_t *>(cur_mask2 + (size_t)I + e);
                if (e < idx_cap) {   // positions the caller expects to be in use (a multiple of 8, or all)
                    v_i0a[w] = *reinterpret_cast<const int4 *>(indices2 + e);
                    v_i0b[w] = *reinterpret_cast<const int4 *>(indices2 + e + 4);
                    v_i1a[w] = *reinterpret_cast<const int4 *>(indices2 + (size_t)I + e);
                    v_i1b[w] = *reinterpret_cast<const int4 *>(indices2 + (size_t)I + e + 4);
                }
            }
        }
        n_both[0] = state[ST_STATE_N_BUF0];
        n_both[1] = state[ST_STATE_N_BUF1];
    }
    after_issue();
    for (int w = tid; w < dirty_words; w += TPB) dirty[w] = 0u;
    const int ep = (int)((tword >> 16) & 1u);
    const bool writer = blockIdx.x == 0;
    pv.ep = ep; pv.writer = writer;

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
                w_cur[w] = nonzero_bytes(ep ? v_cur1[w] : v_cur0[w]);
                if (e < idx_cap) {
                    const int4 a = ep ? v_i1a[w] : v_i0a[w], b4 = ep ? v_i1b[w] : v_i0b[w];
                    uint4 packed;
                    packed.x = (uint32_t)(a.x & 0xffff) | ((uint32_t)a.y << 16);
                    packed.y = (uint32_t)(a.z & 0xffff) | ((uint32_t)a.w << 16);
                    packed.z = (uint32_t)(b4.x & 0xffff) | ((uint32_t)b4.y << 16);
                    packed.w = (uint32_t)(b4.z & 0xffff) | ((uint32_t)b4.w << 16);
                    *reinterpret_cast<uint4 *>(idx_l + e) = packed;
                }
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
    sync();
    after_fill();
    ST_TL(2);
    if (VEC && n > idx_cap) {   // more positions in use than the caller expected: fetch the rest (one more round trip)
        const int32_t *indices = indices2 + (size_t)ep * I;
        for (int p = idx_cap + tid; p < n; p += TPB) idx_l[p] = (uint16_t)indices[p];
        sync();
    }
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
    const uint32_t off = block_excl_scan<TPB / kWave>(cnt, wave_tot, &total, tid, sync);  // contains __syncthreads
    ST_TL(3);
    const int na = (int)(total & 0xffffu), nr = (int)(total >> 16);
    if (na == 0 && nr == 0) {  // unchanged mask: nothing is touched (weight_cache.h:237-240)
        if (tid == 0 && writer) {
            state[ST_STATE_N_CHANGED] = 0;
            state[ST_STATE_N_ADDED] = 0;
            state[ST_STATE_N_REMOVED] = 0;
        }
        pv.next_epoch = ep;
        if (tid == 0) pv.arrival = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
        pv.changed = false;
        pv.n_old = pv.n_new = n; pv.na = pv.nr = 0; pv.n_changed = 0;
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
    sync();

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
            if (MARK || !fast) atomicOr(&dirty[p >> 5], 1u << (p & 31));
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
    sync();

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
        sync();
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
        uint32_t coff = block_excl_scan<TPB / kWave>((uint32_t)__popc(word), wave_tot, &n_changed, tid, sync);  // barrier: lists are dead now
        while (word) {
            const int bit = __ffs(word) - 1;
            word &= word - 1;
            lists[coff++] = (uint16_t)((tid << 5) + bit);
        }
        sync();
    }

    ST_TL(5);
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
    pv.next_epoch = ep ^ 1;
    if (tid == 0) pv.arrival = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
    pv.changed = true;
    pv.n_old = n; pv.n_new = n_new; pv.na = na; pv.nr = nr; pv.n_changed = n_changed;
}


// Last step of a kernel that ran cache_plan: the block that arrived last resets the arrivals and sets the
// epoch.  Looking at the atomic's result only here keeps its round trip off the critical path.
__device__ __forceinline__ void plan_finish(const PlanView &pv, int32_t *__restrict__ state)
{
    if (pv.arriver) {
        uint32_t arrival = pv.arrival;
        asm volatile("" : "+v"(arrival));   // the result is first looked at here, not where it was requested
        if ((arrival & 0xffffu) == gridDim.x - 1)
            atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)pv.next_epoch << 16);
    }
}

// update = plan + this block's share of the row copies
template <bool VEC, int TPB>
__global__ __launch_bounds__(TPB) void cache_update_kernel(const uint8_t *__restrict__ new_mask,
                                                                    uint8_t *__restrict__ cur_mask2,
                                                                    int32_t *__restrict__ indices2,
                                                                    int32_t *__restrict__ state, int I, int gs_log2,
                                                                    int idx_cap, CopyPlan cp)
{
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ PlanShared ps;
    const int tid = threadIdx.x;
    PlanView pv;
    cache_plan<VEC, TPB, false>(pv, smem, &ps, new_mask, cur_mask2, indices2, state, I, idx_cap, tid, [] {}, [] {});
    if (!pv.changed) {
        plan_finish(pv, state);
        return;
    }
    const uint16_t *lists = pv.lists, *idx_l = pv.idx_l;
    const uint32_t n_changed = pv.n_changed;
    const bool writer = pv.writer;
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

    plan_finish(pv, state);
    ST_TL(6);
}

// ---------------------------------------------------------------------------
// update + sparse MLP in ONE kernel, with the plan worked out per POSITION
// instead of per index.
//
// A block only has to know, for each of the <= ceil(I / G) positions it owns,
// which row to read: position p held index e before the update; if e left the
// mask it is the i-th removed index (i = its rank among the removed, ascending)
// and the position receives the i-th added index (weight_cache.h:248-277);
// positions n_old .. n_new-1 receive the surplus additions in ascending order
// (:280-307).  Ranks come from bitmaps of the two masks and per-word prefix
// counts (one wave, no block-wide scans), the i-th added index from a binary
// search over those counts -- no index -> position map, no lists, no atomics,
// three LDS-only barriers, and straight-line code, so the rows a block requests
// on the caller's guess right after its (few) bookkeeping loads stay in flight
// through all of it.  Every block publishes its own positions of the new
// ordered list and a slice of the remembered mask into the other bookkeeping
// buffer; block 0 writes the state words; the last block to arrive flips the
// epoch (as in cache_plan).
// When removals outnumber additions, the surplus ones are taken out one by
// one in the reference (:310-353); their outcome is worked out in closed form
// (see the kernel), or, for very many of them, by cache_plan above for that
// launch only.
// ---------------------------------------------------------------------------
constexpr int kSparseMaxQ = 64;       // positions a block can own
constexpr int kSparseMaxW32 = 512;    // mask words: I <= 16384
constexpr int kSparseWords = 2;       // 8-byte mask words per thread, at most
constexpr int kSparseScan = 4;         // positions per thread whose old index is fetched up front for that replay
constexpr int kSrcPool = 0x40000000;  // src[]: bit 30 = read the pool row (low bits) and write it back; else active row

struct SparseShared {
    uint32_t newbits[kSparseMaxW32], oldbits[kSparseMaxW32];
    uint16_t pr[kSparseMaxW32];   // removed indices below each word
    int na, nr, n;
    int src[kSparseMaxQ];
    int found, paired_tail, replay_ok, fast_ok, nchg;   // surplus removals (removed > added)
};

// 0x01-per-element bytes -> 8 bits (element k -> bit k)
__device__ __forceinline__ uint32_t pack_bits8(uint64_t ones)
{
    return (uint32_t)((ones * 0x0102040810204080ull) >> 56);
}

template <typename T, int RB, int TPB, int NB = 1, int NW = 1, int SPECN = RB / 2>
__global__ __launch_bounds__(TPB) void cache_sparse_decode_kernel(
    const uint8_t *__restrict__ new_mask, uint8_t *__restrict__ cur_mask2, int32_t *__restrict__ indices2,
    int32_t *__restrict__ state, int I, int launch_word, const T *__restrict__ x, int H, int n_hint,
    T *__restrict__ combined, long ldc, float *__restrict__ partials, int act, int plan_bytes, FusedRows fr)
{
    constexpr int VEC = Elem<T>::kVec;
    // Slots of the first batch that are requested ahead of the plan, on the caller's guess of the count and from the
    // active buffers.  A slot whose row turns out to have changed is requested again into the same registers, which
    // has to wait until its first request has arrived; requests return in order, so for the last slots that wait
    // would be the whole stream plus one more round trip, and every row requested in vain is traffic.  The later
    // slots are therefore requested after the plan (first, so that they queue right behind the rows already
    // requested).  Half the batch ahead of the plan measured best (against a third, two thirds and all of it).
    constexpr int SPEC = SPECN;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ float red[TPB / kWave][RB][NB][2];  // per-wave partial (g,u)
    __shared__ float hs[TPB / kWave][RB][NB];      // h of the rows being computed
    __shared__ SparseShared sh;
    __shared__ PlanShared plan_shared;

    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    // (what the first loads need comes first in the argument list, the number of blocks included: the first 14 dwords
    // of the arguments are in scalar registers when the wave starts, anything else -- the launch dimensions too --
    // arrives by a load that the first instructions would wait for.  Four small numbers share one of those dwords.)
    const int blk = blockIdx.x;
    const int G = launch_word & 0xffff, gs_log2 = (launch_word >> 16) & 15, B = (launch_word >> 24) & 15;
    const int chunks = H / VEC;
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    const int GS = 1 << gs_log2, ngrp = TPB >> gs_log2, wpg = GS >> 6;
    const int grp = tid >> gs_log2, cc = tid & (GS - 1);
    const bool valid = cc < chunks;
    const size_t coff = valid ? (size_t)cc * 16 : 0;
    const bool wave_live = __builtin_amdgcn_readfirstlane(cc & ~(kWave - 1)) < chunks;
    const bool has_gate = ((launch_word >> 20) & 1) != 0;
    const int row_bytes = H * (int)sizeof(T);
    const unsigned char *const pool_g = fr.pool_g, *const pool_u = fr.pool_u, *const pool_d = fr.pool_d;
    unsigned char *const act_g = fr.act_g, *const act_u = fr.act_u, *const act_d = fr.act_d;
    const int Q = (I + G - 1) / G;        // positions of this block: blk + G * q, q < Q (host: Q <= kSparseMaxQ)
    const int W32 = (I + 31) >> 5;

    ST_TL(0);
    // ---- bookkeeping loads: one round trip, all unconditional (clamped addresses).  The state words are read
    // through a lane offset the compiler cannot see through (always zero): as loads from one address for the whole
    // wave they would be moved to scalar registers at once, which means waiting for them before anything else
    // is requested.
    int lane_zero = 0;
    asm volatile("" : "+v"(lane_zero));
    const int32_t *state_v = state + lane_zero;
    const uint32_t tword = __hip_atomic_load(reinterpret_cast<const uint32_t *>(&state_v[ST_STATE_TICKET]),
                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int n_buf0 = state_v[ST_STATE_N_BUF0], n_buf1 = state_v[ST_STATE_N_BUF1];
    const int serial_old = state_v[ST_STATE_SERIAL];
    constexpr int nw_rt = NW;   // 8-byte mask words per thread (host: I <= 8 * TPB * NW)
    uint64_t v_new[NW], v_c0[NW], v_c1[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const int e = (tid * nw_rt + w) * 8;
        const int ec = e + 8 <= I ? e : I - 8;
        v_new[w] = *reinterpret_cast<const uint64_t *>(new_mask + ec);
        v_c0[w] = *reinterpret_cast<const uint64_t *>(cur_mask2 + ec);
        v_c1[w] = *reinterpret_cast<const uint64_t *>(cur_mask2 + (size_t)I + ec);
    }
    // The plan is worked out by ONE wave, the last of the block (with 6 KB rows a wave that owns no columns), while
    // the others already request rows; its lanes own the block's positions.
    constexpr int PW = TPB / kWave - 1;
    const bool plan_wave = wave == PW;
    static_assert(kSparseMaxQ == kWave, "one lane of the planning wave per position of the block");
    const int my_p = blk + G * lane;
    const int my_pc = my_p < I ? my_p : I - 1;
    const int i_old0 = indices2[my_pc], i_old1 = indices2[(size_t)I + my_pc];
    // The ordered list itself, four positions per thread, for the case that removals outnumber additions (the
    // surplus ones can sit at any position); only as far as the caller's guess of the count plus a quarter.
    const int n_spec = n_hint < I ? n_hint : I;
    int scan_cap = (n_spec + (n_spec >> 2) + 64) & ~3;
    if (scan_cap > kSparseScan * TPB) scan_cap = kSparseScan * TPB;
    if (scan_cap > I) scan_cap = I & ~3;
    const int scan_p = kSparseScan * tid;
    const bool scan_in = scan_p + kSparseScan <= scan_cap;
    const int scan_pc = scan_in ? scan_p : 0;
    static_assert(kSparseScan == 4, "one 16-byte load per bookkeeping buffer");
    const int4 sc0 = *reinterpret_cast<const int4 *>(indices2 + scan_pc);
    const int4 sc1 = *reinterpret_cast<const int4 *>(indices2 + (size_t)I + scan_pc);
    uint4 xr[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b)
        xr[b] = ld16(reinterpret_cast<const unsigned char *>(x) + (size_t)(b < B ? b : 0) * row_bytes + coff);

    // ---- the first batch of rows, on the caller's guess of the count, from the active buffers
    auto row_of = [&](int bat, int k) { return blk + G * (grp + ngrp * (bat * RB + k)); };
    uint4 wg[RB], wu[RB], wd[RB];
    // (every wave issues the same number of loads whatever its role: a wave without columns, and the gate loads
    // of an ungated cache, read one line of x instead -- with branches around the loads the compiler could no
    // longer tell how many requests are younger than the bookkeeping loads and would wait for all of them)
    // Addresses are a uniform base (scalar registers) plus a 32-bit lane offset, one offset per row for its three
    // matrices: with a 64-bit address per load the 18 requests alone would need 36 registers more.
    const uint32_t coff32 = (uint32_t)coff;
    const unsigned char *const dummy = reinterpret_cast<const unsigned char *>(x);
    const unsigned char *const sp_u = wave_live ? act_u : dummy, *const sp_d = wave_live ? act_d : dummy,
                        *const sp_g = wave_live && has_gate ? act_g : dummy;
    auto speculate = [&](auto lo_c, auto hi_c) __attribute__((always_inline)) {
        constexpr int LO = decltype(lo_c)::value, HI = decltype(hi_c)::value;
#pragma unroll
        for (int k = LO; k < HI; ++k) {
            const int p = row_of(0, k);
            // (a slot past the expected count reads one 16-byte piece for the whole wave: a single request instead of
            // a row's worth of traffic that nobody needs)
            const uint32_t off = wave_live && p < n_spec ? (uint32_t)p * (uint32_t)row_bytes + coff32 : 0u;
            wu[k] = ld16_stream(sp_u + off);
            wd[k] = ld16_stream(sp_d + off);
            wg[k] = ld16_stream(sp_g + (has_gate ? off : 0u));   // (the stand-in line of x has no rows to index)
        }
    };
    // Half of the rows that are requested ahead of the plan go out right behind the bookkeeping loads -- few enough
    // that the memory system is not yet saturated when those loads are served -- the other half once they have
    // arrived.  The barrier only orders the issue: every wave's bookkeeping loads are queued before any wave's rows.
    constexpr int SPEC_A = SPEC / 2;
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    speculate(std::integral_constant<int, 0>{}, std::integral_constant<int, SPEC_A>{});
    __builtin_amdgcn_sched_barrier(0);
    ST_TL(1);

    // ---- masks -> bitmaps in LDS
    const int ep = (int)((tword >> 16) & 1u);
    const int n_old = ep ? n_buf1 : n_buf0;
    uint64_t w_new[NW], w_cur[NW];
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        const int bi = tid * nw_rt + w;            // byte of the bitmaps = elements [8 bi, 8 bi + 8)
        const bool in = w < nw_rt && bi * 8 < I;
        w_new[w] = in ? nonzero_bytes(v_new[w]) : 0ull;
        w_cur[w] = in ? nonzero_bytes(ep ? v_c1[w] : v_c0[w]) : 0ull;
        if (w < nw_rt && bi < W32 * 4) {
            reinterpret_cast<uint8_t *>(sh.newbits)[bi] = (uint8_t)pack_bits8(w_new[w]);
            reinterpret_cast<uint8_t *>(sh.oldbits)[bi] = (uint8_t)pack_bits8(w_cur[w]);
        }
    }
    // (behind the list of added indices, which holds I entries at most; the region of the per-index plan, six
    // bytes per index, is unused on this path)
    uint16_t *const scan_idx = reinterpret_cast<uint16_t *>(smem) + ((I + 7) & ~7);
    if (scan_in) {
        const int4 sc = ep ? sc1 : sc0;
        *reinterpret_cast<uint2 *>(scan_idx + scan_p) =
            make_uint2((uint32_t)(sc.x & 0xffff) | ((uint32_t)sc.y << 16), (uint32_t)(sc.z & 0xffff) | ((uint32_t)sc.w << 16));
    }
    lds_barrier();
    // ---- Rows are requested from here on, i.e. once every wave's bookkeeping loads have ARRIVED: loads issued into
    // a memory system that is already saturated with row requests take several times longer to come back (measured:
    // 5.7 us instead of under 2 when the rows were requested right behind them), and the plan hangs on them.  From
    // here on the plan needs LDS only.  It is one wave's work, so that it does not wait for the other waves either:
    // a wave's requests are accepted only as fast as the memory system takes them (the last wave of sixteen gets its
    // first batch out 3 us after the first), and a block barrier inside the plan would wait for all of that.
    ST_TL(2);
    int n = n_old;      // count after the update
    uint32_t arrival = 0;
    __builtin_amdgcn_sched_barrier(0);
    if (plan_wave) {
        // ---- per-word prefix counts of added / removed indices, eight words per lane at most
        const int wpl = (W32 + kWave - 1) >> 6;
        // (words per lane: at most 4 per 8-byte mask word a thread reads -- the host launches NW = 1 up to I = 8192 --
        // so that the unrolled loops below are no longer than this launch needs: the code of this branch is run by one
        // wave per block, once, and what it costs is mostly fetching it)
        constexpr int kWpl = 4 * NW;
        static_assert(kWpl * kWave * 32 >= 8 * TPB * NW, "the planning wave covers every mask word of the launch");
        uint32_t la[kWpl], lr[kWpl], aw[kWpl];
        uint32_t ca = 0, cr = 0;
        // (all reads of the bitmaps are issued together, from clamped addresses; the words stay in registers for the
        // second pass)
        uint32_t nwd[kWpl], owd[kWpl];
#pragma unroll
        for (int j = 0; j < kWpl; ++j) {
            const int t = lane * wpl + j;
            const int tc = t < W32 ? t : W32 - 1;
            nwd[j] = sh.newbits[tc];
            owd[j] = sh.oldbits[tc];
        }
#pragma unroll
        for (int j = 0; j < kWpl; ++j) {
            const int t = lane * wpl + j;
            const bool in = j < wpl && t < W32;
            const uint32_t nw = in ? nwd[j] : 0u, ow = in ? owd[j] : 0u;
            la[j] = ca; lr[j] = cr;
            aw[j] = nw & ~ow;
            ca += (uint32_t)__popc(aw[j]);
            cr += (uint32_t)__popc(ow & ~nw);
        }
        const uint32_t packed = ca | (cr << 16);
        const uint32_t incl = wave_incl_scan_dpp(packed, lane);
        const uint32_t excl = incl - packed;
        // removed: per-word prefix counts (a position looks its old index's rank up); added: the ascending list itself
        uint16_t *added_list = reinterpret_cast<uint16_t *>(smem);   // (the region of the per-index plan, unused on this path)
#pragma unroll
        for (int j = 0; j < kWpl; ++j) {
            const int t = lane * wpl + j;
            if (j < wpl && t < W32) {
                sh.pr[t] = (uint16_t)((excl >> 16) + lr[j]);
                // (a word rarely holds more than two added indices: the first two go out without a loop)
                uint32_t a = aw[j];
                int o = (int)((excl & 0xffffu) + la[j]);
                const uint32_t a2 = a & (a - 1u);
                if (a) added_list[o] = (uint16_t)(t * 32 + __ffs((int)a) - 1);
                if (a2) added_list[o + 1] = (uint16_t)(t * 32 + __ffs((int)a2) - 1);
                a = a2 & (a2 - 1u);
                o += 2;
                while (a) {
                    added_list[o++] = (uint16_t)(t * 32 + __ffs((int)a) - 1);
                    a &= a - 1u;
                }
            }
        }
        const uint32_t tot = (uint32_t)__builtin_amdgcn_readlane((int)incl, kWave - 1);
        const int na_w = (int)(tot & 0xffffu), nr_w = (int)(tot >> 16);
        // (LDS operations of one wave execute in order: the lanes below read what other lanes of this wave wrote above)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
        int s = -1;
        if (nr_w <= na_w) {
            // ---- every removed index is paired with an added one: the positions' sources follow per position
            int nn = n_old + (na_w - nr_w);
            if (nn > I) nn = I;
            if (lane < Q && my_p < nn) {
                int newidx;
                if (my_p < n_old) {
                    const int e = ep ? i_old1 : i_old0;
                    const int word = (e >> 5) & (kSparseMaxW32 - 1), bit = e & 31;
                    const uint32_t remw = sh.oldbits[word] & ~sh.newbits[word];
                    if ((remw >> bit) & 1u) {
                        const int rank = (int)sh.pr[word] + __popc(remw & ((1u << bit) - 1u));
                        newidx = (int)added_list[rank];
                        s = newidx | kSrcPool;
                    } else {
                        newidx = e;
                        s = my_p;
                    }
                } else {
                    newidx = (int)added_list[nr_w + (my_p - n_old)];
                    s = newidx | kSrcPool;
                }
                if ((na_w | nr_w) != 0) indices2[(size_t)(ep ^ 1) * I + my_p] = newidx;
            }
            if (lane == 0) sh.n = nn;
        } else {
            // ---- Removals outnumber additions: the surplus ones are taken out one by one, in ascending index order,
            // each by moving the last entry of the list into its place (weight_cache.h:310-353).  With S of them the list
            // ends as its first n_old - S positions ("base"); step k moves the entry that sits in tail slot S-1-k at
            // that time to where the k-th surplus index sits at that time.  Only the tail (S entries of the list, fetched
            // up front) has to be looked at: a surplus index that starts below the tail stays where it is until its own
            // step, so the lane that owns its position asks what step k moves ("land[k]"), and if that is another
            // surplus index (one that started in the tail and is taken out later), what that one's step moves, and
            // so on.  Inside the tail the moves depend on each other through the surplus indices that START there
            // (few: about S^2 / n_old): their slot at their own step is resolved first, one lane each, in rounds (a
            // lane whose chase runs into one that is not resolved yet tries again; the smallest always gets through);
            // then every entry of the tail follows the moves until a step takes it below the tail.  All of it is this
            // wave's work: the others keep streaming.  Used when S <= min(256, I/4), at most 64 surplus indices start
            // in the tail and the list was fetched far enough up front; else the whole block works it out behind the
            // barrier (below), or the per-index plan does.
            const int S = nr_w - na_w, base = n_old - S;   // uniform
            const int smax_w = (I >> 2) < TPB ? (I >> 2) : TPB;
            const int sm8 = (smax_w + 7) & ~7;
            constexpr int kMark = 0x8000, kNone = 0xffff, kOut = 0xfffe, kPop = 0xfffd, kUnres = 0xfffc;
            // (LDS behind the list of added indices: the fetched list, then five arrays of smax entries: 6.5 bytes per index at most)
            uint16_t *const loc = scan_idx + ((scan_cap + 7) & ~7);   // k -> tail slot the k-th surplus index starts in
            uint16_t *const tailv = loc + sm8;                        // tail slot -> entry after the paired replacements, or kMark | k
            uint16_t *const jres = tailv + sm8;                       // k (starting in the tail) -> its slot at step k
            uint16_t *const land = jres + sm8;                        // k -> what step k moves below the tail
            uint16_t *const jlist = land + sm8;                       // the surplus indices that start in the tail
            // (S <= 256: one wave walks the tail 64 slots at a time, and beyond four passes the whole block is faster)
            bool ok = S <= smax_w && S <= 4 * kWave && base >= 0 && n_old <= scan_cap && I >= 256;
            if (ok) {
#pragma unroll 1
                for (int c = lane; c < S; c += kWave) loc[c] = (uint16_t)kNone;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                int in_tail = 0, paired_tail = 0;
#pragma unroll 1
                for (int c = 0; c < S; c += kWave) {
                    const int j = c + lane;
                    const bool in = j < S;
                    const int e = (int)scan_idx[base + (in ? j : 0)];
                    const int word = (e >> 5) & (kSparseMaxW32 - 1), bit = e & 31;
                    const uint32_t remw = sh.oldbits[word] & ~sh.newbits[word];
                    const bool rem = in && ((remw >> bit) & 1u);
                    const int rank = (int)sh.pr[word] + __popc(remw & ((1u << bit) - 1u));
                    const bool paired = rem && rank < na_w, extra = rem && rank >= na_w;
                    const int k = extra ? rank - na_w : 0;
                    int v = e;
                    if (paired) v = (int)added_list[rank];
                    if (extra) v = kMark | k;
                    if (in) tailv[j] = (uint16_t)v;
                    const uint64_t mx = __builtin_amdgcn_ballot_w64(extra);
                    if (extra) {
                        const int jj = in_tail + __popcll(mx & ((1ull << lane) - 1ull));
                        loc[k] = (uint16_t)j;
                        jres[k] = (uint16_t)kUnres;
                        if (jj < kWave) jlist[jj] = (uint16_t)k;
                    }
                    in_tail += __popcll(mx);
                    paired_tail += __popcll(__builtin_amdgcn_ballot_w64(paired));
                }
                ok = in_tail <= kWave;
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                if (ok) {
                    // ---- the surplus indices that start in the tail: where each sits at its own step
                    const int kk = lane < in_tail ? (int)jlist[lane] : -1;
                    bool open = kk >= 0;
#pragma unroll 1
                    for (int round = 0; round <= kWave && __builtin_amdgcn_ballot_w64(open) != 0; ++round) {
                        bool done = false;
                        int res = 0;
                        if (open) {
                            int pos = loc[kk];
#pragma unroll 1
                            for (int it = 0; it <= S; ++it) {
                                const int i = S - 1 - pos;   // the step that takes the entry of that slot
                                if (i > kk) { res = pos; done = true; break; }    // still there at its own step
                                if (i == kk) { res = kPop; done = true; break; }  // the last entry at its own step: nothing moves
                                const int li = loc[i], ji = jres[i];
                                if (li == kNone || ji == kOut) {   // step i moves it below the tail
                                    land[i] = (uint16_t)(kMark | kk);
                                    res = kOut; done = true; break;
                                }
                                if (ji == kUnres) break;   // next round
                                pos = ji;                  // step i moved it to that slot
                            }
                        }
                        if (open && done) jres[kk] = (uint16_t)res;
                        open = open && !done;
                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                        __builtin_amdgcn_wave_barrier();
                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                    }
                    // ---- every other entry of the tail follows the moves until one takes it below the tail
#pragma unroll 1
                    for (int c = lane; c < S; c += kWave) {
                        const int v = tailv[c];
                        if (v & kMark) continue;
                        int k = S - 1 - c;
#pragma unroll 1
                        for (int it = 0; it <= S; ++it) {
                            const int lk = loc[k], jk = jres[k];
                            if (lk == kNone || jk == kOut) { land[k] = (uint16_t)v; break; }
                            k = S - 1 - (jk < S ? jk : 0);
                        }
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                    if (lane < Q && my_p < base) {
                        const int e = ep ? i_old1 : i_old0;
                        const int word = (e >> 5) & (kSparseMaxW32 - 1), bit = e & 31;
                        const uint32_t remw = sh.oldbits[word] & ~sh.newbits[word];
                        int newidx = e;
                        if ((remw >> bit) & 1u) {
                            const int rank = (int)sh.pr[word] + __popc(remw & ((1u << bit) - 1u));
                            if (rank < na_w) {
                                newidx = (int)added_list[rank];
                            } else {
                                int v = land[(rank - na_w) < S ? rank - na_w : 0];
#pragma unroll 1
                                for (int it = 0; it < S && (v & kMark); ++it) v = land[(v & (kMark - 1)) < S ? (v & (kMark - 1)) : 0];
                                newidx = v < I ? v : e;   // (consistent bookkeeping always ends at an entry of the list)
                            }
                        }
                        s = newidx != e ? (newidx | kSrcPool) : my_p;
                        indices2[(size_t)(ep ^ 1) * I + my_p] = newidx;
                    }
                    if (lane == 0) {
                        sh.n = base;
                        // rewritten positions: the pairs' below the tail, and the places of the surplus indices below it
                        sh.nchg = na_w - paired_tail + (S - in_tail);
                    }
                }
            }
            if (lane == 0) sh.fast_ok = ok ? 1 : 0;
        }
        sh.src[lane] = s;
        if (lane == 0) { sh.na = na_w; sh.nr = nr_w; sh.found = 0; sh.paired_tail = 0; }
    }
    speculate(std::integral_constant<int, SPEC_A>{}, std::integral_constant<int, SPEC>{});
    __builtin_amdgcn_sched_barrier(0);
    lds_barrier();
    ST_TL(3);
    const int na = sh.na, nr = sh.nr;
    const bool changed = (na | nr) != 0;
    bool arriver = plan_wave && lane == 0;
    int next_epoch = ep;
    // Removals outnumber additions: the surplus ones are taken out one by one, in ascending index order, each by
    // moving the last entry of the list into its place (weight_cache.h:310-353).  With S of them the list ends as
    // its first n_old - S positions ("base"); the entries of the last S positions ("tail") that stay end up in the
    // places of the surplus indices below the tail.  Step k takes the entry at tail slot S-1-k and puts it where
    // the k-th surplus index sits at that time: its place in the list, unless that place is a tail slot whose own
    // step came earlier (then it has travelled on with that step's move, possibly again).  So the places follow
    // from the start positions by chasing through tail slots, which only surplus indices that START in the tail
    // need (few: about S^2 / n_old); they are resolved one after the other, then every surviving tail entry finds
    // its final place on its own.  This is the whole block's form of it, for the case that more than 64 surplus
    // indices start in the tail (the planning wave has done the others on its own, `fast`).  Used when
    // S <= min(1024, I/4) and the list was fetched far enough up front; else the per-index plan.
    const int surplus = nr - na, tail_base = n_old - surplus;
    const bool fast = surplus > 0 && sh.fast_ok != 0;
    const int smax = (I >> 2) < TPB ? (I >> 2) : TPB;
    // (LDS behind the list of added indices: the fetched list, then five arrays of smax entries: 6.5 bytes per index at most)
    bool replay = surplus > 0 && !fast && surplus <= smax && tail_base >= 0 && n_old <= scan_cap && I >= 256;
    constexpr uint16_t kGone = 0xffffu;   // hole[]: removed as the last entry, nothing moves; tailv[]: a surplus index
    uint16_t *const hole = scan_idx + ((scan_cap + 7) & ~7);   // start position of the k-th surplus index, then its place at step k
    uint16_t *const tailv = hole + ((smax + 7) & ~7);          // entry of tail slot j after the paired replacements
    if (replay) {
        const uint16_t *added_list = reinterpret_cast<const uint16_t *>(smem);
        // ---- every thread, four positions: paired replacements in place; where the surplus indices sit; the tail
        if (scan_in && scan_p < n_old) {
            uint2 pk = *reinterpret_cast<const uint2 *>(scan_idx + scan_p);
            uint32_t ent[kSparseScan] = {pk.x & 0xffffu, pk.x >> 16, pk.y & 0xffffu, pk.y >> 16};
            int found = 0, paired_tail = 0;
#pragma unroll
            for (int j = 0; j < kSparseScan; ++j) {
                const int p = scan_p + j;
                const int e = (int)ent[j];
                if (p < n_old) {
                    const int word = (e >> 5) & (kSparseMaxW32 - 1), bit = e & 31;
                    const uint32_t remw = sh.oldbits[word] & ~sh.newbits[word];
                    const bool rem = (remw >> bit) & 1u;
                    const int rank = rem ? (int)sh.pr[word] + __popc(remw & ((1u << bit) - 1u)) : 0;
                    const bool extra = rem && rank >= na;
                    if (rem && !extra) ent[j] = added_list[rank];
                    if (extra) { hole[rank - na] = (uint16_t)p; ++found; }
                    if (p >= tail_base) {
                        tailv[p - tail_base] = extra ? kGone : (uint16_t)ent[j];
                        if (rem && !extra) ++paired_tail;
                    }
                }
            }
            pk.x = ent[0] | (ent[1] << 16); pk.y = ent[2] | (ent[3] << 16);
            *reinterpret_cast<uint2 *>(scan_idx + scan_p) = pk;
            if (found) atomicAdd(&sh.found, found);
            if (paired_tail) atomicAdd(&sh.paired_tail, paired_tail);
        }
        lds_barrier();
        // ---- one wave: the places of the surplus indices that start in the tail.  An index's place depends on those
        // of smaller surplus indices only, and only on such that start in the tail themselves (the others stay where
        // they are), so they are resolved 64 at a time, one lane each, in rounds: a lane whose chase runs into an
        // index that is not resolved yet tries again in the next round (the smallest unresolved one always gets
        // through; two or three rounds as a rule).
        if (plan_wave) {
            const int S = __builtin_amdgcn_readfirstlane(surplus), base = __builtin_amdgcn_readfirstlane(tail_base);
            uint16_t *const jlist = tailv + ((smax + 7) & ~7);   // [S] the surplus indices (their rank k) that start in the tail
            uint16_t *const jrank = jlist + ((smax + 7) & ~7);   // [S] k -> position in jlist
            uint16_t *const jres = jrank + ((smax + 7) & ~7);    // [S] k -> resolved place
            int in_tail = 0;
            for (int c = 0; c < S; c += kWave) {
                const int k = c + lane;
                const bool is = k < S && (int)hole[k < S ? k : 0] >= base;
                const uint64_t m = __builtin_amdgcn_ballot_w64(is);
                if (is) {
                    const int j = in_tail + __popcll(m & ((1ull << lane) - 1ull));
                    jlist[j] = (uint16_t)k;
                    jrank[k] = (uint16_t)j;
                }
                in_tail += __popcll(m);
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
            for (int j0 = 0; j0 < in_tail; j0 += kWave) {
                const int kk = j0 + lane < in_tail ? (int)jlist[j0 + lane] : -1;
                bool open = kk >= 0;
                uint64_t resolved = 0;   // lanes of this group that are done (the same in every lane)
                int place = 0;
                for (int round = 0; round <= kWave && __builtin_amdgcn_ballot_w64(open) != 0; ++round) {
                    bool done = false;
                    if (open) {
                        int pos = hole[kk];
                        for (int it = 0; it <= S; ++it) {
                            const int i = S - 1 - (pos - base);   // the step that takes the entry of that tail slot
                            if (pos < base || pos == (int)kGone || i > kk || i < 0) { done = true; break; }   // stays there
                            if (i == kk) { pos = kGone; done = true; break; }   // it is the last entry at its own step
                            const int h = hole[i];
                            if (h < base) { pos = h; done = true; break; }      // travelled with an index that never moves
                            const int j = jrank[i];
                            if (j >= j0 && !((resolved >> (j - j0)) & 1ull)) break;   // not known yet: next round
                            pos = jres[i];
                        }
                        place = pos;
                    }
                    const uint64_t now = __builtin_amdgcn_ballot_w64(open && done);
                    if (open && done) jres[kk] = (uint16_t)place;
                    resolved |= now;
                    open = open && !done;
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
                }
            }
            // (hole[] kept the start positions until here: the chase tells the two kinds of surplus index apart by them)
            for (int j = lane; j < in_tail; j += kWave) {
                const int kk = jlist[j];
                hole[kk] = jres[kk];
            }
            if (lane == 0) {
                // (a surplus index missing from the list would make the counts disagree: per-index plan then)
                sh.replay_ok = sh.found == S;
                sh.n = base;
                // rewritten positions: the pairs' below the tail, and the places of the surplus indices below it
                sh.nchg = na - sh.paired_tail + (S - in_tail);
            }
        }
        lds_barrier();
        replay = sh.replay_ok != 0;
        if (replay) {
            // ---- every surviving tail entry to its final place
            if (tid < surplus) {
                const uint16_t v = tailv[tid];
                if (v != kGone) {
                    int pos = hole[surplus - 1 - tid];
                    for (int it = 0; it < surplus && pos >= tail_base && pos < n_old; ++it)
                        pos = hole[surplus - 1 - (pos - tail_base)];
                    if (pos < tail_base) scan_idx[pos] = v;
                }
            }
            lds_barrier();
            if (plan_wave) {
                int s = -1;
                if (lane < Q && my_p < tail_base) {
                    const int newidx = scan_idx[my_p];
                    s = newidx != (ep ? i_old1 : i_old0) ? (newidx | kSrcPool) : my_p;
                    indices2[(size_t)(ep ^ 1) * I + my_p] = newidx;
                }
                sh.src[lane] = s;
            }
            lds_barrier();
        }
    }
    if (surplus <= 0 || fast || replay) {
        const int n_changed = fast || replay ? sh.nchg : na;
        n = sh.n;
        if (changed) {
            // the remembered mask: 8-byte words dealt to the blocks round-robin (the reference keeps the old
            // mask when the update leaves nothing active)
            uint8_t *mask_out = cur_mask2 + (size_t)(ep ^ 1) * I;
#pragma unroll
            for (int w = 0; w < NW; ++w) {
                const int bi = tid * nw_rt + w;
                if (w < nw_rt && bi * 8 < I && (bi % G) == blk)
                    *reinterpret_cast<uint64_t *>(mask_out + (size_t)bi * 8) = n > 0 ? w_new[w] : w_cur[w];
            }
            if (blk == 0 && arriver) {
                state[ST_STATE_N_BUF0 + (ep ^ 1)] = n;
                state[ST_STATE_N_ACTIVE] = n;
                state[ST_STATE_N_CHANGED] = n_changed;
                state[ST_STATE_N_ADDED] = na;
                state[ST_STATE_N_REMOVED] = nr;
                state[ST_STATE_SERIAL] = serial_old + 1;
                state[ST_STATE_EPOCH] = ep ^ 1;
                if (n > 0) {
                    state[ST_STATE_STATUS] = 0;
                    state[ST_STATE_VALID] = 1;
                } else {
                    state[ST_STATE_STATUS] = ST_ERR_NO_ACTIVE;
                }
            }
            next_epoch = ep ^ 1;
        } else if (blk == 0 && arriver) {
            state[ST_STATE_N_CHANGED] = 0;
            state[ST_STATE_N_ADDED] = 0;
            state[ST_STATE_N_REMOVED] = 0;
        }
        if (arriver) arrival = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
    } else {
        // ---- too many surplus removals for the replay above: the per-index plan
        PlanView pv;
        cache_plan<true, TPB, true>(pv, smem, &plan_shared, new_mask, cur_mask2, indices2, state, I, I, tid,
                                           [] {}, [] {});
        n = pv.n_new;
        if (plan_wave) {
            int s = -1;
            if (lane < Q && my_p < n) {
                const bool moved = my_p >= pv.n_old || ((pv.dirty[my_p >> 5] >> (my_p & 31)) & 1u);
                s = moved ? ((int)pv.idx_l[my_p] | kSrcPool) : my_p;
            }
            sh.src[lane] = s;
        }
        arriver = pv.arriver; arrival = pv.arrival; next_epoch = pv.next_epoch;
        // (requested again so that the first request's registers are free while the plan above runs)
        speculate(std::integral_constant<int, 0>{}, std::integral_constant<int, SPEC>{});
        lds_barrier();
    }
    ST_TL(4);

    float acc[NB][VEC];
#pragma unroll
    for (int b = 0; b < NB; ++b)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[b][e] = 0.f;

    const int jcount = n > blk ? (n - blk + G - 1) / G : 0;      // rows of this block
    const int nbat = ((jcount + ngrp - 1) / ngrp + RB - 1) / RB;  // uniform over the block
    for (int bat = 0; bat < nbat; ++bat) {
        unsigned fresh = 0u;   // bit k: row of slot k comes from the pool and has to be written back
        auto request = [&](int k, bool speculated) __attribute__((always_inline)) {
            const int q = grp + ngrp * (bat * RB + k);
            const int p = blk + G * q;
            const int s = sh.src[q < kSparseMaxQ ? q : kSparseMaxQ - 1];
            const bool ok = q < Q && s >= 0;
            const bool pooled = ok && (s & kSrcPool) != 0;
            if (pooled) fresh |= 1u << k;
            if (speculated && !pooled && p < n_spec) return;
            const size_t ro = ok ? (size_t)(s & (kSrcPool - 1)) * row_bytes + coff : 0;   // no row: one piece for the whole wave
            wu[k] = ld16_stream((pooled ? pool_u : act_u) + ro);
            wd[k] = ld16_stream((pooled ? pool_d : act_d) + ro);
            wg[k] = has_gate ? ld16_stream((pooled ? pool_g : act_g) + ro) : zero4;
        };
        if (wave_live) {
            const bool spec = bat == 0 && n_spec > 0;
#pragma unroll
            for (int k = SPEC; k < RB; ++k) request(k, false);
#pragma unroll
            for (int k = 0; k < SPEC; ++k) request(k, spec);
            if (spec && !has_gate) {
#pragma unroll
                for (int k = 0; k < SPEC; ++k) wg[k] = zero4;
            }
        } else {
#pragma unroll
            for (int k = 0; k < RB; ++k) wg[k] = wu[k] = wd[k] = zero4;
        }
        ST_TL(6);

        // ---- phase 1: partial dot products on this thread's chunk
        uint4 xq[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) xq[b] = (valid && b < B) ? xr[b] : zero4;
#pragma unroll
        for (int k = 0; k < RB; ++k) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float pg = 0.f, pu = 0.f;
                dot_chunk<T>(wg[k], wu[k], xq[b], pg, pu);
                const float sg = wave_sum_dpp(pg), su = wave_sum_dpp(pu);
                if (lane == 0) {
                    red[wave][k][b][0] = sg;
                    red[wave][k][b][1] = su;
                }
            }
        }
        // write the fresh rows back while the reductions settle
#pragma unroll
        for (int k = 0; k < RB; ++k) {
            if (((fresh >> k) & 1u) && valid) {
                const size_t ro = (size_t)row_of(bat, k) * row_bytes + coff;
                st16(act_u + ro, wu[k]);
                st16(act_d + ro, wd[k]);
                if (has_gate) st16(act_g + ro, wg[k]);
            }
        }
        __syncthreads();
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
        // ---- phase 2: down projection from the rows already in registers
#pragma unroll
        for (int k = 0; k < RB; ++k) {
            const bool row_ok = row_of(bat, k) < n;
            const uint4 rd = row_ok ? wd[k] : zero4;
#pragma unroll
            for (int b = 0; b < NB; ++b) axpy_chunk<T>(hs[grp][k][b], rd, acc[b]);
        }
    }

    // ---- combine the thread groups through LDS (behind the plan arrays), one fp32 partial row per block
    if (ngrp > 1) {
        float *redc = reinterpret_cast<float *>(smem + plan_bytes);  // [ngrp-1][NB][H]
        if (grp > 0 && valid) {
#pragma unroll
            for (int b = 0; b < NB; ++b)
#pragma unroll
                for (int e = 0; e < VEC; e += 4)
                    *reinterpret_cast<float4 *>(redc + ((size_t)(grp - 1) * NB + b) * H + (size_t)cc * VEC + e) =
                        make_float4(acc[b][e], acc[b][e + 1], acc[b][e + 2], acc[b][e + 3]);
        }
        __syncthreads();
        if (grp == 0 && valid) {
            for (int gq = 1; gq < ngrp; ++gq)
#pragma unroll
                for (int b = 0; b < NB; ++b)
#pragma unroll
                    for (int e = 0; e < VEC; e += 4) {
                        const float4 v = *reinterpret_cast<const float4 *>(redc + ((size_t)(gq - 1) * NB + b) * H +
                                                                            (size_t)cc * VEC + e);
                        acc[b][e] += v.x; acc[b][e + 1] += v.y; acc[b][e + 2] += v.z; acc[b][e + 3] += v.w;
                    }
        }
    }
    if (grp == 0 && valid) {
#pragma unroll
        for (int b = 0; b < NB; ++b)
#pragma unroll
            for (int e = 0; e < VEC; e += 4)
                *reinterpret_cast<float4 *>(partials + ((size_t)blk * NB + b) * H + (size_t)cc * VEC + e) =
                    make_float4(acc[b][e], acc[b][e + 1], acc[b][e + 2], acc[b][e + 3]);
    }
    // the block that arrived last resets the arrivals and sets the epoch (the atomic's result is first looked at here)
    if (arriver) {
        asm volatile("" : "+v"(arrival));
        if ((arrival & 0xffffu) == (uint32_t)G - 1u)
            atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)next_epoch << 16);
    }
    ST_TL(7);
}

// ---------------------------------------------------------------------------
// update for intermediate sizes the kernels above cannot hold in LDS (kPlanMaxI < I <= kBigMaxI).
// The same replay of WeightCache::update_active_weights (weight_cache.h:229-359) in every block, with the
// masks as bitmaps and no added / removed lists: the i-th removed or added index is found through per-word
// prefix counts (rank of a set bit; i-th set bit by bisection), which leaves 4.5 bytes of LDS per element --
// the two index maps the sequential surplus removals (:310-353) need.  Blocks then copy the rows of the
// positions they own (position p belongs to block p mod (blocks - 1); block 0 publishes the bookkeeping).
// ---------------------------------------------------------------------------
constexpr int64_t kBigMaxI = 32768;
constexpr int kBigThreads = 1024;
constexpr int kBigWords = 4;   // 8-byte mask words per thread: I <= 8 * 1024 * 4

constexpr size_t big_lds_bytes(int I)
{
    const size_t w32 = (size_t)((I + 31) >> 5);
    return (size_t)I * 4 + w32 * 4 * 3 + w32 * 2 * 2 + 64;
}

struct BigShared {
    uint32_t wave_tot[kBigThreads / kWave];
    int n_new, na, nr;
};

// index of the i-th (from 0) set bit of bits[w] & ~mask_out[w] over all words, given the exclusive prefix counts
__device__ __forceinline__ int big_select(const uint32_t *bits, const uint32_t *notbits, const uint16_t *prefix, int W32, int i)
{
    int lo = 0;
    for (int step = 1024; step >= 1; step >>= 1) {
        const int c = lo + step;
        if (c < W32 && (int)prefix[c] <= i) lo = c;
    }
    uint32_t w = bits[lo] & ~notbits[lo];
    int j = i - (int)prefix[lo], pos = 0;
#pragma unroll
    for (int half = 16; half >= 1; half >>= 1) {
        const uint32_t lowmask = (1u << half) - 1u;
        const int c = __popc(w & lowmask);
        if (j >= c) { j -= c; pos += half; w >>= half; }
        w &= lowmask;
    }
    return lo * 32 + pos;
}

__global__ __launch_bounds__(kBigThreads) void cache_update_big_kernel(const uint8_t *__restrict__ new_mask,
                                                                      uint8_t *__restrict__ cur_mask2,
                                                                      int32_t *__restrict__ indices2,
                                                                      int32_t *__restrict__ state, int I, FusedRows fr)
{
    constexpr int TPB = kBigThreads;
    extern __shared__ __align__(16) unsigned char smem[];
    __shared__ BigShared bs;
    const int tid = threadIdx.x;
    const int W32 = (I + 31) >> 5;
    uint16_t *pos_l = reinterpret_cast<uint16_t *>(smem);   // index -> position (kNone when absent)
    uint16_t *idx_l = pos_l + I;                            // position -> index
    uint32_t *newbits = reinterpret_cast<uint32_t *>(idx_l + I + (I & 1));
    uint32_t *oldbits = newbits + W32, *dirty = oldbits + W32;
    uint16_t *pa = reinterpret_cast<uint16_t *>(dirty + W32), *pr = pa + W32 + (W32 & 1);
    auto sync = [&]() __attribute__((always_inline)) { lds_barrier(); };

    const uint32_t tword = __hip_atomic_load(reinterpret_cast<const uint32_t *>(&state[ST_STATE_TICKET]), __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_AGENT);
    const int ep = (int)((tword >> 16) & 1u);
    const int n = state[ST_STATE_N_BUF0 + ep];
    const int serial_old = state[ST_STATE_SERIAL];
    const uint8_t *cur_mask = cur_mask2 + (size_t)ep * I;
    const int32_t *indices = indices2 + (size_t)ep * I;
    // masks -> bitmaps (8 elements per byte of the bitmaps), kept as 0x01 bytes in registers for publishing
    uint64_t w_new[kBigWords], w_cur[kBigWords];
#pragma unroll
    for (int w = 0; w < kBigWords; ++w) {
        const int bi = tid * kBigWords + w;
        const bool in = bi * 8 < I;
        const int ec = in ? bi * 8 : 0;
        w_new[w] = in ? nonzero_bytes(*reinterpret_cast<const uint64_t *>(new_mask + ec)) : 0ull;
        w_cur[w] = in ? nonzero_bytes(*reinterpret_cast<const uint64_t *>(cur_mask + ec)) : 0ull;
        if (bi < W32 * 4) {
            reinterpret_cast<uint8_t *>(newbits)[bi] = (uint8_t)pack_bits8(w_new[w]);
            reinterpret_cast<uint8_t *>(oldbits)[bi] = (uint8_t)pack_bits8(w_cur[w]);
        }
    }
    for (int i = tid; i < I; i += TPB) pos_l[i] = kNone;
    for (int w = tid; w < W32; w += TPB) dirty[w] = 0u;
    for (int p = tid; p < n; p += TPB) idx_l[p] = (uint16_t)indices[p];
    sync();
    for (int p = tid; p < n; p += TPB) pos_l[idx_l[p]] = (uint16_t)p;
    // per-word prefix counts of added / removed indices (one word per thread: W32 <= 1024)
    uint32_t addw = 0u, remw = 0u;
    if (tid < W32) { addw = newbits[tid] & ~oldbits[tid]; remw = oldbits[tid] & ~newbits[tid]; }
    uint32_t total;
    const uint32_t off = block_excl_scan<TPB / kWave>((uint32_t)__popc(addw) | ((uint32_t)__popc(remw) << 16), bs.wave_tot,
                                                      &total, tid, sync);
    if (tid < W32) { pa[tid] = (uint16_t)(off & 0xffffu); pr[tid] = (uint16_t)(off >> 16); }
    const int na = (int)(total & 0xffffu), nr = (int)(total >> 16);
    const bool writer = blockIdx.x == 0;
    uint32_t arrival = 0;
    if (na == 0 && nr == 0) {   // unchanged mask: nothing is touched (weight_cache.h:237-240)
        if (tid == 0 && writer) {
            state[ST_STATE_N_CHANGED] = 0;
            state[ST_STATE_N_ADDED] = 0;
            state[ST_STATE_N_REMOVED] = 0;
        }
        if (tid == 0) {
            arrival = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
            if ((arrival & 0xffffu) == gridDim.x - 1)
                atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)ep << 16);
        }
        return;
    }
    sync();   // pos_l, pa, pr complete
    const int pairs = na < nr ? na : nr;
    // ---- phase 1: the i-th removed index hands its position to the i-th added one; phase 2: surplus additions appended
    if (tid < W32) {
        uint32_t r = remw;
        int rank = (int)pr[tid];
        while (r && rank < pairs) {
            const int e = tid * 32 + __ffs((int)r) - 1;
            r &= r - 1u;
            const uint16_t p = pos_l[e];
            if (p != kNone) {
                const int a = big_select(newbits, oldbits, pa, W32, rank);
                idx_l[p] = (uint16_t)a;
                pos_l[a] = p;
                pos_l[e] = kNone;
                atomicOr(&dirty[p >> 5], 1u << (p & 31));
            }
            ++rank;
        }
        uint32_t a_bits = addw;
        int arank = (int)pa[tid];
        while (a_bits) {
            const int a = tid * 32 + __ffs((int)a_bits) - 1;
            a_bits &= a_bits - 1u;
            if (arank >= pairs) {
                const int p = n + (arank - pairs);
                if (p < I) {
                    idx_l[p] = (uint16_t)a;
                    pos_l[a] = (uint16_t)p;
                    atomicOr(&dirty[p >> 5], 1u << (p & 31));
                }
            }
            ++arank;
        }
    }
    sync();
    int n_new;
    if (nr <= na) {
        n_new = n + (na - pairs);
        if (n_new > I) n_new = I;
    } else {
        // ---- phase 3: surplus removals in ascending index order, sequential by construction
        if (tid == 0) {
            int m = n, k = 0;
            for (int w = 0; w < W32; ++w) {
                uint32_t r = oldbits[w] & ~newbits[w];
                while (r) {
                    const int e = w * 32 + __ffs((int)r) - 1;
                    r &= r - 1u;
                    if (k++ < pairs) continue;
                    const uint16_t p = pos_l[e];
                    if (p == kNone) continue;
                    if (m <= 0) { w = W32; break; }
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
            }
            bs.n_new = m;
        }
        sync();
        n_new = bs.n_new;
    }
    // rows rewritten: positions below the new count whose index changed
    uint32_t dcount = 0;
    for (int w = tid; w < W32; w += TPB) {
        uint32_t d = dirty[w];
        const int lo = w << 5;
        if (lo >= n_new) d = 0u;
        else if (lo + 32 > n_new) d &= (1u << (n_new - lo)) - 1u;
        dcount += (uint32_t)__popc(d);
    }
    uint32_t n_changed;
    (void)block_excl_scan<TPB / kWave>(dcount, bs.wave_tot, &n_changed, tid, sync);
    // ---- publish: block 0 writes the other bookkeeping buffer, the last arrival flips the epoch
    if (writer) {
        int32_t *idx_out = indices2 + (size_t)(ep ^ 1) * I;
        uint8_t *mask_out = cur_mask2 + (size_t)(ep ^ 1) * I;
        for (int p = tid; p < n_new; p += TPB) idx_out[p] = idx_l[p];
#pragma unroll
        for (int w = 0; w < kBigWords; ++w) {
            const int bi = tid * kBigWords + w;
            if (bi * 8 < I) *reinterpret_cast<uint64_t *>(mask_out + (size_t)bi * 8) = n_new > 0 ? w_new[w] : w_cur[w];
        }
        if (tid == 0) {
            state[ST_STATE_N_BUF0 + (ep ^ 1)] = n_new;
            state[ST_STATE_N_ACTIVE] = n_new;
            state[ST_STATE_N_CHANGED] = (int)n_changed;
            state[ST_STATE_N_ADDED] = na;
            state[ST_STATE_N_REMOVED] = nr;
            state[ST_STATE_SERIAL] = serial_old + 1;
            state[ST_STATE_EPOCH] = ep ^ 1;
            if (n_new > 0) {
                state[ST_STATE_STATUS] = 0;
                state[ST_STATE_VALID] = 1;
            } else {
                state[ST_STATE_STATUS] = ST_ERR_NO_ACTIVE;
            }
        }
    }
    if (tid == 0) arrival = atomicAdd(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), 1u);
    // ---- copies: active[p] <- pool[index at p] for the dirty positions this block owns
    {
        const int row_bytes = fr.row_bytes, chunks = row_bytes >> 4;
        const bool has_gate = fr.has_gate != 0;
        const bool solo = gridDim.x == 1;
        const int owners = solo ? 1 : (int)gridDim.x - 1, me = solo ? 0 : (int)blockIdx.x - 1;
        if (solo || !writer) {
            for (int p = me; p < n_new; p += owners) {
                if (!((dirty[p >> 5] >> (p & 31)) & 1u)) continue;   // uniform over the block
                const size_t from = (size_t)idx_l[p] * row_bytes, to = (size_t)p * row_bytes;
                for (int c = tid; c < chunks; c += TPB) {
                    const size_t o = (size_t)c << 4;
                    const uint4 vu = ld16(fr.pool_u + from + o), vd = ld16(fr.pool_d + from + o);
                    uint4 vg = make_uint4(0u, 0u, 0u, 0u);
                    if (has_gate) vg = ld16(fr.pool_g + from + o);
                    st16(fr.act_u + to + o, vu);
                    st16(fr.act_d + to + o, vd);
                    if (has_gate) st16(fr.act_g + to + o, vg);
                }
            }
        }
    }
    if (tid == 0 && (arrival & 0xffffu) == gridDim.x - 1)
        atomicExch(reinterpret_cast<uint32_t *>(&state[ST_STATE_TICKET]), (uint32_t)(ep ^ 1) << 16);
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

extern "C" int64_t st_cache_max_intermediate(void) { return st::kBigMaxI; }

extern "C" st_cache *st_cache_create(const st_cache_buffers *bufs, int64_t I, int64_t H, int dtype, int has_gate)
{
    using namespace st;
    auto fail = [](const char *m) -> st_cache * { set_error("st_cache_create: %s", m); return nullptr; };
    if (!bufs) return fail("null buffers");
    if (dtype < ST_F32 || dtype > ST_BF16) return fail("unknown dtype");
    const int esz = dtype == ST_F32 ? 4 : 2;
    if (I < 1 || I > kBigMaxI) return fail("intermediate size out of range (see st_cache_max_intermediate)");
    if (I > kPlanMaxI && I % 8 != 0) return fail("intermediate sizes above 22000 must be multiples of 8");
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
    for (int i = 0; i < ST_STATE_WORDS; ++i) c->host_state[i] = 0;
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
    if (I > kPlanMaxI) {   // index maps of the other kernels do not fit the LDS: bitmap plan, rows by position
        ST_REQUIRE(I % 8 == 0 && (uintptr_t)mask % 8 == 0 && (uintptr_t)c->b.cur_mask % 8 == 0,
                   "st_cache_update_async: for I > %lld the masks must be 8-byte aligned", (long long)kPlanMaxI);
        FusedRows fr;
        fr.pool_u = static_cast<const unsigned char *>(c->b.up_pool);
        fr.act_u = static_cast<unsigned char *>(c->b.up_active);
        fr.pool_d = static_cast<const unsigned char *>(c->b.downT_pool);
        fr.act_d = static_cast<unsigned char *>(c->b.down_active);
        fr.pool_g = c->has_gate ? static_cast<const unsigned char *>(c->b.gate_pool) : fr.pool_u;
        fr.act_g = c->has_gate ? static_cast<unsigned char *>(c->b.gate_active) : fr.act_u;
        fr.row_bytes = (int)(c->H * c->esz);
        fr.has_gate = c->has_gate ? 1 : 0;
        const size_t lds_big = big_lds_bytes(I);
        static std::atomic<bool> big_attr{false};
        if (!big_attr.load(std::memory_order_acquire)) {
            ST_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(cache_update_big_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 156 * 1024));
            big_attr.store(true, std::memory_order_release);
        }
        ProfScope ps(ST_K_CACHE_UPDATE, s);
        ST_LAUNCH(ps, cache_update_big_kernel, dim3(device_cu_count()), dim3(kBigThreads), lds_big, s, mask,
                  c->b.cur_mask, c->b.indices, c->b.state, I, fr);
        ST_HIP(hipGetLastError());
        return ST_OK;
    }
    const size_t lds = plan_lds_bytes(I);
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
    const int grid = blocks ? blocks : device_cu_count() * 3 / 4;   // (measured against 1/4, 3/8, 1/2 and all of the CUs)
    const bool aligned = (I % 8 == 0) && ((uintptr_t)mask % 8 == 0) && ((uintptr_t)c->b.cur_mask % 8 == 0) &&
                         ((uintptr_t)c->b.indices % 16 == 0);
    // 512-thread blocks (ST_CACHE_TPB=512) leave room on the CU for a kernel of another stream, but
    // measure slower on their own; they cover I <= 12288 in the vector path.
    const bool small = want_tpb == 512 && aligned && I <= 8 * 512 * kPlanMaxWords;
    const int tpb = small ? 512 : 1024;
    const bool vec = aligned && I <= 8 * tpb * kPlanMaxWords;
    int gs_log2 = 6;
    while ((1 << gs_log2) < chunks && (1 << gs_log2) < tpb) ++gs_log2;
    // how much of the index list the blocks fetch up front: a quarter more than the count the host saw
    // last (st_cache_sync_state), everything when it has seen none
    const int seen = c->host_state[ST_STATE_N_ACTIVE];
    const int idx_cap = seen > 0 && seen + seen / 4 + 64 < I ? (seen + seen / 4 + 64 + 7) & ~7 : I;
    {
        ProfScope ps(ST_K_CACHE_UPDATE, s);
        auto launch = [&](auto kern) -> int {
            const int arc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), 160 * 1024 - 256);
            if (arc != ST_OK) return arc;
            ST_LAUNCH(ps, kern, dim3(grid), dim3(tpb), lds, s, mask, c->b.cur_mask, c->b.indices, c->b.state,
                               I, gs_log2, idx_cap, cp);
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

extern "C" int st_cache_update_forward(st_cache *c, const uint8_t *mask, const void *x, int64_t B, int64_t n_hint,
                                       void *out, void *combined, int64_t ldc, void *workspace,
                                       int64_t workspace_bytes, int act, void *stream)
{
    using namespace st;
    ST_REQUIRE(c && mask && x && out && workspace, "st_cache_update_forward: null pointer");
    ST_REQUIRE(B >= 1 && B <= 4096, "st_cache_update_forward: B=%lld out of range [1,4096]", (long long)B);
    ST_REQUIRE(act >= ST_ACT_RELU && act <= ST_ACT_IDENTITY, "st_cache_update_forward: unknown activation %d", act);
    ST_REQUIRE(workspace_bytes >= st_mlp_workspace_bytes(B, c->H, c->I),
               "st_cache_update_forward: workspace too small (%lld < %lld)", (long long)workspace_bytes,
               (long long)st_mlp_workspace_bytes(B, c->H, c->I));
    ST_REQUIRE((((uintptr_t)x | (uintptr_t)workspace) & 15) == 0, "st_cache_update_forward: pointers must be 16-byte aligned");
    // the count after the update is only known on the device: `combined` has to hold the largest possible one
    ST_REQUIRE(!combined || ldc >= (c->has_gate ? 2 : 1) * c->I,
               "st_cache_update_forward: ldc=%lld too small for %lld intermediate rows", (long long)ldc, (long long)c->I);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int I = (int)c->I, H = (int)c->H;
    const int row_bytes = (int)(c->H * c->esz), chunks = row_bytes >> 4;
    constexpr int TPB = 1024;
    int gs_log2 = 6;
    while ((1 << gs_log2) < chunks && (1 << gs_log2) < TPB) ++gs_log2;
    const int ngrp = TPB >> gs_log2;
    const size_t plan_bytes = (plan_lds_bytes(I) + 15) & ~(size_t)15;
    const int NBF = B == 2 ? 2 : 1;   // rows of x the fused kernel takes in one pass
    const size_t lds = plan_bytes + (size_t)(ngrp - 1) * NBF * H * 4;
    const int G = mlp_grid();
    const bool aligned = (I % 8 == 0) && ((uintptr_t)mask % 8 == 0) && ((uintptr_t)c->b.cur_mask % 8 == 0) &&
                         ((uintptr_t)c->b.indices % 16 == 0);
    static const bool fused_off = [] { const char *v = getenv("ST_CACHE_FUSED"); return v && atoi(v) == 0; }();
    // One kernel for one or two rows of x when a block owns at most kSparseMaxQ positions, the masks fit the
    // kernel's bitmaps and a row fits one pass of a thread group; everything else runs as two calls.
    const bool fused = !fused_off && B <= 2 && aligned && I >= 8 && G <= 0xffff && (I + G - 1) / G <= kSparseMaxQ &&
                       I <= 32 * kSparseMaxW32 && I <= 8 * TPB * kSparseWords && chunks <= TPB && row_bytes % 16 == 0 &&
                       lds <= (size_t)(148 * 1024);
    if (!fused) {   // two launches: update, then the forward that reads the count on the device
        const int rc = st_cache_update_async(c, mask, stream);
        if (rc != ST_OK) return rc;
        return st_mlp_forward(x, B, c->H, c->b.gate_active, c->b.up_active, c->b.down_active, c->I,
                              c->b.state + ST_STATE_N_ACTIVE, n_hint, out, combined, ldc, workspace, workspace_bytes, act,
                              c->dtype, c->has_gate, stream);
    }
    FusedRows fr;
    fr.pool_u = static_cast<const unsigned char *>(c->b.up_pool);
    fr.act_u = static_cast<unsigned char *>(c->b.up_active);
    fr.pool_d = static_cast<const unsigned char *>(c->b.downT_pool);
    fr.act_d = static_cast<unsigned char *>(c->b.down_active);
    fr.pool_g = c->has_gate ? static_cast<const unsigned char *>(c->b.gate_pool) : fr.pool_u;
    fr.act_g = c->has_gate ? static_cast<unsigned char *>(c->b.gate_active) : fr.act_u;
    fr.row_bytes = row_bytes;
    fr.has_gate = c->has_gate ? 1 : 0;
    float *partials = static_cast<float *>(workspace);
    const int hint = (int)(n_hint < 0 ? 0 : (n_hint > c->I ? c->I : n_hint));
    {
        ProfScope ps(ST_K_CACHE_UPDATE_DECODE, s);
        auto launch = [&](auto kern, auto *xt, auto *ct) -> int {
            const int arc = allow_dynamic_lds(reinterpret_cast<const void *>(kern), 148 * 1024);
            if (arc != ST_OK) return arc;
            // (blocks, log2 of the thread-group size, gated or not, rows of x: one argument, see the kernel)
            const int launch_word = G | (gs_log2 << 16) | (fr.has_gate << 20) | ((int)B << 24);
            ST_LAUNCH(ps, kern, dim3(G), dim3(TPB), lds, s, mask, c->b.cur_mask, c->b.indices, c->b.state, I,
                      launch_word, xt, H, hint, ct, (long)ldc, partials, act, (int)plan_bytes, fr);
            return ST_OK;
        };
        int rc;
        // Rows a thread group keeps in flight (it does not change which rows a group sums, or in which order): six;
        // seven where the caller's guess of the count gives a group 7, 13 or 14 rows (one batch less); three when
        // a group has at most three rows; two rows of x: six when that is one batch, else five.
        const int rpg = ((hint + G - 1) / G + ngrp - 1) / ngrp;   // rows per thread group on the caller's guess
        const bool seven = c->dtype != ST_F32 && B == 1 && (rpg + 6) / 7 < (rpg + 5) / 6;
#define ST_SPARSE_NW(TYPE, ROWS, NBX)                                                                               \
    rc = I <= 8 * TPB ? launch(cache_sparse_decode_kernel<TYPE, ROWS, TPB, NBX, 1>, xt, ct)                         \
                      : launch(cache_sparse_decode_kernel<TYPE, ROWS, TPB, NBX, 2>, xt, ct)
// (three rows in flight: two of them ahead of the plan -- with so few rows per block nearly everything waits for the plan
// otherwise; measured +4 % tok/s on the 10 %-active workloads against one, and against all three)
#define ST_SPARSE_NW3(TYPE)                                                                                         \
    rc = I <= 8 * TPB ? launch(cache_sparse_decode_kernel<TYPE, 3, TPB, 1, 1, 2>, xt, ct)                           \
                      : launch(cache_sparse_decode_kernel<TYPE, 3, TPB, 1, 2, 2>, xt, ct)
#define ST_SPARSE_LAUNCH(TYPE)                                                                                      \
    do {                                                                                                            \
        const TYPE *xt = static_cast<const TYPE *>(x);                                                              \
        TYPE *ct = static_cast<TYPE *>(combined);                                                                   \
        if (B == 2 && rpg <= 6) ST_SPARSE_NW(TYPE, 6, 2);                                                           \
        else if (B == 2) ST_SPARSE_NW(TYPE, 5, 2);                                                                  \
        else if (seven) ST_SPARSE_NW(TYPE, 7, 1);                                                                   \
        else if (rpg >= 1 && rpg <= 3) ST_SPARSE_NW3(TYPE);                                                         \
        else ST_SPARSE_NW(TYPE, DecodeRows<TYPE>::value, 1);                                                        \
    } while (0)
        if (c->dtype == ST_F32) ST_SPARSE_LAUNCH(float);
        else if (c->dtype == ST_BF16) ST_SPARSE_LAUNCH(bf16_t);
        else ST_SPARSE_LAUNCH(f16_t);
#undef ST_SPARSE_LAUNCH
#undef ST_SPARSE_NW
#undef ST_SPARSE_NW3
        if (rc != ST_OK) return rc;
    }
    ST_HIP(hipGetLastError());
    return launch_mlp_reduce(c->dtype, partials, G, NBF, (int)B, H, out, s);
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
    if (c->host_state[ST_STATE_FAULT] != 0) {
        set_error("st_cache: the fault word of the state is set; the cache contents are undefined");
        return ST_ERR_HIP;
    }
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
