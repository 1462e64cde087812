/*
 * sparse_mlp_amd.h — C ABI of the MI355X (gfx950) sparse-MLP decode path.
 *
 * Plain pointers and sizes only: every `const void*` / `void*` below is a
 * DEVICE pointer unless its comment says "host"; `stream` is a hipStream_t
 * passed as void* (NULL = the default stream).  All entry points return
 * ST_OK (0) or a negative st_status; st_last_error() gives a message for the
 * calling thread.  No entry point except st_cache_create/st_cache_destroy
 * (host memory only) and st_cache_sync_state (one small device-to-host copy)
 * allocates or synchronises: work is enqueued on `stream` and ordered with
 * whatever else the caller enqueues there.
 *
 * Each entry point names the interface of NimbleEdge/sparse_transformers it
 * replaces (paths relative to that repository).
 */
#ifndef SPARSE_MLP_AMD_H
#define SPARSE_MLP_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum st_status {
    ST_OK = 0,
    ST_ERR_ARG = -1,       /* bad shape / alignment / null pointer / unsupported size */
    ST_ERR_NO_ACTIVE = -2, /* update left the cache empty: the reference's "No active weights" */
    ST_ERR_HIP = -3,       /* a HIP runtime call failed */
    ST_ERR_INVALID = -4    /* cache has no valid contents yet: the reference's "Cache is not valid" */
} st_status;

/* ST_F64: st_mlp_forward only (the reference's operator is dtype-generic, sparse_mlp_op.cpp:151-161, and its CUDA
 * kernels are instantiated for double, sparse_mlp_cuda.cu:90-151); caches and the predictor take the first three. */
typedef enum st_dtype { ST_F32 = 0, ST_F16 = 1, ST_BF16 = 2, ST_F64 = 3 } st_dtype;

typedef enum st_act {
    ST_ACT_RELU = 0,      /* what sparse_mlp_op.cpp:157,183 computes */
    ST_ACT_SILU = 1,      /* ACT2FN["silu"], src/modeling_skip.py:65,116 */
    ST_ACT_GELU_TANH = 2, /* "gelu_pytorch_tanh" (gemma3n) */
    ST_ACT_SIGMOID = 3,   /* what sparse_mlp_cuda.cu:83 computes */
    ST_ACT_IDENTITY = 4
} st_act;

int st_version(void);
/* host; message of the last failing call made by this thread ("" if none) */
const char *st_last_error(void);

/* ------------------------------------------------------------------------
 * Sparse MLP forward.
 * Replaces sparse_mlp_forward / sparse_mlp_forward_cpu
 * (sparse_transformers/csrc/sparse_mlp_op.cpp:53-76,79-192), the Python path
 * SkipMLP._forward_sparse_weight_cache (src/modeling_skip.py:114-117) and the
 * ungated OPTSkipMLP variant (src/models/opt/modelling_opt_skip.py:116-119).
 *
 *   x          [B,H]   activations, dtype `dtype`
 *   gate_rows  [n,H]   active gate rows (NULL when !has_gate): concat_weight[:n]
 *   up_rows    [n,H]   active up rows: concat_weight[n:2n] (concat_weight when ungated)
 *   down_rows  [n,H]   active down columns, packed one per row: the memory
 *                      behind active_down_weight ([H,n], strides (1,H))
 *   n                  host-side active count; rows >= n are never read
 *   n_dev              optional device int32: when non-NULL the kernels use
 *                      min(*n_dev, n) instead, so a cache update and the
 *                      forward can be enqueued back to back with no host read
 *                      (rows in [*n_dev, n) may be read but are ignored, so
 *                      the buffers must really hold n rows)
 *   n_hint             only with n_dev: the count the host expects (0 = no
 *                      idea).  Rows below it are requested before *n_dev has
 *                      arrived and it picks how many rows stay in flight; a
 *                      wrong hint costs time, never correctness
 *   out        [B,H]   dtype `dtype`   (the reference's down_proj_buffer)
 *   combined   [B,ldc] dtype `dtype`, optional (NULL = skip): receives
 *                      act(gate)*up in columns [0,n) and, when gated, the raw
 *                      up projection in [n,2n) — what the in-place operator
 *                      leaves in combined_proj_buffer
 *   workspace          scratch of st_mlp_workspace_bytes(B,H,n) bytes
 * All rows must be 16-byte aligned (H*sizeof(dtype) % 16 == 0). B <= 4096.
 * B <= 2 (and any B < 32 in fp32 or with a hidden size the MFMA kernels do not
 * cover) runs the streaming decode kernel; 3 <= B <= 32 in fp16 / bf16 with
 * H % 256 == 0 (H <= 16384) runs the MFMA batch kernels (still HBM-bound; one
 * pass over the weights per 32 rows of x for H in {2048, 3072, 4096}, per 16
 * rows otherwise); otherwise B >= 32 in fp16 / bf16 with H % 128 == 0
 * runs the MFMA GEMM kernels (then only columns [0,n) of `combined` carry results; when its rows are 16-byte
 * aligned and have room, the kernels keep their intermediate there and also zero the columns from n up to the next
 * multiple of 128).
 * ST_F64 (any B, H % 2 == 0): three plain kernels with every sum in double and in a fixed order, eight rows of x
 * per pass; the workspace must then hold st_mlp_f64_workspace_bytes(B,H,n) bytes.
 * ------------------------------------------------------------------------ */
int64_t st_mlp_workspace_bytes(int64_t B, int64_t H, int64_t n);
int64_t st_mlp_f64_workspace_bytes(int64_t B, int64_t H, int64_t n);
int st_mlp_forward(const void *x, int64_t B, int64_t H, const void *gate_rows, const void *up_rows,
                   const void *down_rows, int64_t n, const int32_t *n_dev, int64_t n_hint, void *out, void *combined,
                   int64_t ldc, void *workspace, int64_t workspace_bytes, int act, int dtype, int has_gate,
                   void *stream);

/* The same forward for callers that cannot allocate or bring a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Arguments as for
 * st_mlp_forward without the workspace; only B <= 2 (the streaming decode
 * kernel).  The fp32 partial rows go to a scratch array that is part of the
 * library image (st_mlp_static_scratch_bytes() = 8 MiB per GPU, resident until
 * the process ends); a call needs blocks * B * H * 4 bytes of it (one block per
 * CU) and is refused with ST_ERR_ARG beyond that.  Every element the reduction
 * reads is written by the same call first, so nothing has to be cleared between
 * calls.  All calls on one GPU share the array: calls that overlap in time on
 * the same GPU (two streams, two threads) race.  No hipMalloc / hipFree or
 * other allocating call is made. */
int64_t st_mlp_static_scratch_bytes(void);
int st_mlp_forward_static(const void *x, int64_t B, int64_t H, const void *gate_rows, const void *up_rows,
                          const void *down_rows, int64_t n, const int32_t *n_dev, int64_t n_hint, void *out,
                          void *combined, int64_t ldc, int act, int dtype, int has_gate, void *stream);

/* ------------------------------------------------------------------------
 * LoRA predictor -> threshold mask -> union over rows, on the device.
 * Replaces FastLoRAProjection.forward (src/modeling_skip.py:52-53) and the
 * "naive" branch plus any(dim=0) of SkipDecoderLayer._compute_binary_mask
 * (src/modeling_skip.py:204-207,214), generalised from 0 to a scalar
 * threshold.
 *
 *   x [B,H], A [r,H] (down.weight), Bm [I,r] (up.weight), all dtype `dtype`
 *   t_ws    float [B,r] scratch (the rank-r intermediate, kept in fp32)
 *   scores  optional float [B,I] (NULL = not written)
 *   mask    uint8 [I]: mask[i] = any_b(score[b,i] >= thr)  (cmp_ge != 0)
 *                               any_b(score[b,i] >  thr)  (cmp_ge == 0)
 * H*sizeof(dtype) and r*sizeof(dtype) must be multiples of 16.  More than 64 rows
 * of x (fewer for ranks above 224) run as several passes over the predictor's weights.
 * ------------------------------------------------------------------------ */
int st_predictor_mask(const void *x, int64_t B, int64_t H, const void *A, int64_t r, const void *Bm, int64_t I,
                      int dtype, float thr, int cmp_ge, float *t_ws, float *scores, uint8_t *mask, void *stream);
/* The same with flags.  ST_PRED_ROUND_STORAGE: the rank-r intermediate and the scores are rounded to `dtype` before
 * they are used, which is what FastLoRAProjection computes when the model runs in fp16 / bf16 (up(down(x)) as two
 * modules in the model's type, src/modeling_skip.py:52-53): scores close to the cut then fall on the side the
 * reference's own arithmetic puts them.  Without it both stay in fp32 (st_predictor_mask).  No effect for ST_F32. */
enum st_predictor_flags { ST_PRED_ROUND_STORAGE = 1 };
int st_predictor_mask_ex(const void *x, int64_t B, int64_t H, const void *A, int64_t r, const void *Bm, int64_t I,
                         int dtype, float thr, int cmp_ge, int flags, float *t_ws, float *scores, uint8_t *mask,
                         void *stream);

/* ------------------------------------------------------------------------
 * Mask methods that need a statistic of the whole score row, then the union
 * over rows.  Replaces the "topk" and "statistical_topk" branches and the
 * any(dim=0) of SkipDecoderLayer._compute_binary_mask
 * (src/modeling_skip.py:208-214, _gaussian_topk :197-202).
 *   scores  float [B,I] (what st_predictor_mask leaves in `scores`)
 *   method  ST_MASK_TOPK: per row the k largest scores (equal scores: lower
 *           index first; k <= 0 selects nothing, k >= I everything)
 *           ST_MASK_STATISTICAL: score > mean + std * z per row, population
 *           std, strict >; z = Normal(0,1).icdf(sparsity) in the reference
 *   mask    uint8 [I], union over the B rows
 *   cutoff  optional float [B]: the k-th largest score / the statistical cut
 *   workspace  only for B > 1: st_mask_select_workspace_bytes(B, I) bytes,
 *           16-byte aligned; its first 16 bytes must be zero before the first
 *           call and are left zero by every call.  Calls that share a
 *           workspace must not overlap.
 * ------------------------------------------------------------------------ */
enum st_mask_method { ST_MASK_TOPK = 0, ST_MASK_STATISTICAL = 1 };
int64_t st_mask_select_workspace_bytes(int64_t B, int64_t I);
int st_mask_select(const float *scores, int64_t B, int64_t I, int method, int64_t k, float z, uint8_t *mask,
                   float *cutoff, void *workspace, int64_t workspace_bytes, void *stream);

/* Per-row approximate top-k threshold from four max-sketches.  Replaces
 * approx_topk_threshold (sparse_transformers/csrc/approx_topk.h:10-88, registered
 * in sparse_mlp_op.cpp:208) for float scores: threshold[b] = 0.9 * the
 * max(1, k*cells/F)-th largest sketch cell of row b.  F >= 4, 0 < k <= F. */
int st_approx_topk_threshold(const float *scores, int64_t B, int64_t F, int64_t k, float *threshold, void *stream);
/* The same for double scores and thresholds (the reference dispatches on every floating type, approx_topk.h:33;
 * its adjustment factor is then the double 0.9). */
int st_approx_topk_threshold_f64(const double *scores, int64_t B, int64_t F, int64_t k, double *threshold,
                                 void *stream);

/* ------------------------------------------------------------------------
 * Differential weight cache, resident in HBM.
 * Replaces class WeightCache (sparse_transformers/csrc/weight_cache.h:13-381)
 * as registered in sparse_mlp_op.cpp:198-202.  The caller owns every device
 * buffer (so a torch allocator, or plain hipMalloc, can provide them); the
 * handle only holds host-side bookkeeping.
 * ------------------------------------------------------------------------ */
typedef struct st_cache_buffers {
    /* pools: all rows, never modified after st_cache_load_weights */
    void *gate_pool;   /* [I,H] (NULL when !has_gate) */
    void *up_pool;     /* [I,H] */
    void *downT_pool;  /* [I,H]: row i = column i of the [H,I] down matrix */
    /* packed active rows, capacity I rows each; first n_active rows valid */
    void *gate_active; /* [I,H] (NULL when !has_gate) */
    void *up_active;   /* [I,H] */
    void *down_active; /* [I,H] */
    /* bookkeeping, double-buffered: buffer e lives at offset e*I, the current e is state[ST_STATE_EPOCH] */
    int32_t *indices;  /* [2*I] ordered active list (the reference's active_indices) */
    uint8_t *cur_mask; /* [2*I] the reference's current_mask */
    int32_t *state;    /* [ST_STATE_WORDS] see st_state_word */
} st_cache_buffers;

enum st_state_word {
    ST_STATE_N_ACTIVE = 0,  /* number of valid rows in the active buffers */
    ST_STATE_N_CHANGED = 1, /* rows rewritten by the last update */
    ST_STATE_STATUS = 2,    /* 0 ok, ST_ERR_NO_ACTIVE after an update that emptied the cache */
    ST_STATE_VALID = 3,     /* the reference's cache_valid */
    ST_STATE_N_ADDED = 4,   /* |new & ~old| of the last update */
    ST_STATE_N_REMOVED = 5, /* |old & ~new| of the last update */
    ST_STATE_SERIAL = 6,    /* updates that changed something */
    ST_STATE_EPOCH = 7,     /* which half of indices / cur_mask is current */
    ST_STATE_TICKET = 8,    /* internal: (epoch << 16) | blocks arrived in the running update */
    ST_STATE_N_BUF0 = 9,    /* internal: active count of bookkeeping buffer 0 */
    ST_STATE_N_BUF1 = 10,   /* internal: active count of bookkeeping buffer 1 */
    ST_STATE_FAULT = 11,    /* reserved (no kernel waits on another block any more); nonzero is reported as ST_ERR_HIP */
    ST_STATE_WORDS = 16
};

typedef struct st_cache st_cache;

/* Largest intermediate size the update kernels support (32768: their plan lives in LDS -- index maps up to
 * 22000, bitmaps with two index maps beyond; the reference has no bound, weight_cache.h:167). */
int64_t st_cache_max_intermediate(void);

/* host only.  weight_cache.h:148-194 (allocation is the caller's). */
st_cache *st_cache_create(const st_cache_buffers *bufs, int64_t I, int64_t H, int dtype, int has_gate);
void st_cache_destroy(st_cache *c);

/* Fill the pools (down [H,I] is transposed on the device) and reset the
 * bookkeeping to "nothing active, current_mask = 0": weight_cache.h:199-223.
 * gate/up [I,H], down [H,I], dtype of the cache; gate may be NULL when ungated. */
int st_cache_load_weights(st_cache *c, const void *gate, const void *up, const void *down, void *stream);

/* update_active_weights(mask): weight_cache.h:229-359 (diff :84-110, pairing
 * :248-277, append :280-307, swap-with-last :310-353).  mask: uint8/bool [I]
 * on the device.  Enqueues one kernel (bookkeeping + row copies); returns
 * without waiting.  An update that empties the cache sets
 * state[ST_STATE_STATUS] = ST_ERR_NO_ACTIVE and, like the reference, leaves
 * cur_mask unchanged. */
int st_cache_update_async(st_cache *c, const uint8_t *mask, void *stream);

/* Copies the state words to the host (waits for `stream`).  Returns
 * ST_ERR_NO_ACTIVE if the last update emptied the cache, else ST_OK.
 * state_out: host int32[ST_STATE_WORDS], may be NULL. */
int st_cache_sync_state(st_cache *c, int32_t *state_out, void *stream);

/* update_active_weights(mask) immediately followed by the sparse MLP on the
 * updated cache -- weight_cache.h:229-359 then sparse_mlp_op.cpp:53-192 /
 * src/modeling_skip.py:114-117, i.e. what SkipDecoderLayer.forward does per
 * layer (src/modeling_skip.py:234-261) -- enqueued as one call.  For B <= 2
 * (16-byte aligned rows, 8-byte aligned mask, I % 8 == 0, I <= 16384) this is
 * ONE kernel in which every block works out where the rows of the positions
 * it owns come from and streams them, taking rows whose index changed from
 * the pool and writing them back on the way; otherwise it is
 * st_cache_update_async followed by st_mlp_forward.  Either way the cache
 * ends in the same state and `out` holds the same bits as the two separate
 * calls.  x, out: [B,H] in the cache's dtype; combined: [B,ldc] or NULL;
 * workspace: st_mlp_workspace_bytes(B, H, I) bytes.  n_hint: the active count
 * the host last saw (0 = unknown); it picks the kernel variant, which rows are
 * requested before the plan is known and how much of the index list is
 * fetched up front, and never affects results.  An update that empties
 * the cache leaves status ST_ERR_NO_ACTIVE in the state words (reported by
 * st_cache_sync_state) and zeros in `out`. */
int st_cache_update_forward(st_cache *c, const uint8_t *mask, const void *x, int64_t B, int64_t n_hint, void *out,
                            void *combined, int64_t ldc, void *workspace, int64_t workspace_bytes, int act,
                            void *stream);

/* get_concat_weight(): weight_cache.h:113-145,362-366.  Writes the contiguous
 * [2n,H] (gate rows then up rows; [n,H] when ungated) tensor into dst, for
 * callers that need the reference's tensor; n is the host's count from the
 * last st_cache_sync_state. */
int st_cache_materialize_concat(st_cache *c, void *dst, int64_t n, void *stream);

/* ------------------------------------------------------------------------
 * Per-kernel timing with HIP events, for benchmarks (no counterpart in the
 * reference, whose benchmark.py:149-156 times whole generations from the
 * host).  While enabled, every kernel launched by this library is bracketed
 * by a pair of events recorded on the launch stream; st_profile_collect waits
 * for them and returns one (kind, milliseconds) sample per launch.  Recording
 * costs a few microseconds per launch, so throughput is measured with
 * profiling off.
 * ------------------------------------------------------------------------ */
typedef enum st_kernel_kind {
    ST_K_MLP_DECODE = 0,
    ST_K_MLP_REDUCE = 1,
    ST_K_CACHE_UPDATE = 2,
    ST_K_MASK_SELECT = 3,
    ST_K_PRED_DOWN = 4,
    ST_K_PRED_UP_MASK = 5,
    ST_K_MLP_PREFILL_GATEUP = 6,
    ST_K_MLP_PREFILL_DOWN = 7,
    ST_K_MLP_BATCH_GATEUP = 8,
    ST_K_MLP_BATCH_DOWN = 9,
    ST_K_CACHE_UPDATE_DECODE = 10,
    ST_K_KINDS = 11
} st_kernel_kind;

int st_profile_enable(int max_samples); /* host; allocates the event pool */
int st_profile_disable(void);
/* host; kinds/ms: arrays of `cap` entries; waits for the recorded events and
 * returns the number of samples written (or a negative st_status).  The
 * sample list is kept (st_profile_enable starts a new one), so launches that
 * were captured into a HIP graph can be read again after every replay. */
int st_profile_collect(int *kinds, float *ms, int cap);

#ifdef __cplusplus
}
#endif
#endif /* SPARSE_MLP_AMD_H */
