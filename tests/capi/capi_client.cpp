// A client of the C ABI that uses nothing but the HIP runtime and include/sparse_mlp_amd.h: what a binding
// in another language does.  Builds a small cache from host arrays, runs two updates, the sparse MLP after
// each (once as update + forward, once as the single fused call) and the predictor mask, and checks every
// result against a plain loop over the same arrays: index order as WeightCache::update_active_weights
// leaves it (sparse_transformers/csrc/weight_cache.h:229-359, worked out by hand below), the output of
// sparse_mlp_forward (sparse_transformers/csrc/sparse_mlp_op.cpp:151-161) with the activation in the
// Python path (src/modeling_skip.py:114-117).  Prints "capi_client: OK" and exits 0 on success.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../../include/sparse_mlp_amd.h"

#define HIP_OK(call)                                                                      \
    do {                                                                                  \
        hipError_t e_ = (call);                                                           \
        if (e_ != hipSuccess) {                                                           \
            std::printf("capi_client: %s failed: %s\n", #call, hipGetErrorString(e_));    \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)
#define ST_CALL(call)                                                                     \
    do {                                                                                  \
        int rc_ = (call);                                                                 \
        if (rc_ != ST_OK) {                                                               \
            std::printf("capi_client: %s -> %d (%s)\n", #call, rc_, st_last_error());     \
            return 1;                                                                     \
        }                                                                                 \
    } while (0)

static float silu(float v) { return v / (1.f + std::exp(-v)); }

template <typename T> static T *to_device(const std::vector<T> &h)
{
    T *d = nullptr;
    if (hipMalloc(&d, h.size() * sizeof(T)) != hipSuccess) return nullptr;
    if (hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
    return d;
}

int main()
{
    const int I = 16, H = 8, r = 4;   // H * 4 bytes = 32: rows are 16-byte multiples
    std::vector<float> gate(I * H), up(I * H), down(H * I), A(r * H), Bm(I * r), x(H);
    uint32_t seed = 12345u;
    auto rnd = [&] { seed = seed * 1664525u + 1013904223u; return ((seed >> 8) & 0xffff) / 65536.f - 0.5f; };
    for (auto *v : {&gate, &up, &down, &A, &Bm, &x})
        for (float &f : *v) f = rnd();

    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    float *d_gate = to_device(gate), *d_up = to_device(up), *d_down = to_device(down), *d_x = to_device(x);
    float *d_A = to_device(A), *d_Bm = to_device(Bm);
    if (!d_gate || !d_up || !d_down || !d_x || !d_A || !d_Bm) { std::printf("capi_client: device alloc failed\n"); return 1; }

    // ---- the cache: every device buffer is the caller's
    st_cache_buffers bufs{};
    const size_t mat = (size_t)I * H * sizeof(float);
    HIP_OK(hipMalloc(&bufs.gate_pool, mat)); HIP_OK(hipMalloc(&bufs.up_pool, mat)); HIP_OK(hipMalloc(&bufs.downT_pool, mat));
    HIP_OK(hipMalloc(&bufs.gate_active, mat)); HIP_OK(hipMalloc(&bufs.up_active, mat)); HIP_OK(hipMalloc(&bufs.down_active, mat));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&bufs.indices), 2 * I * sizeof(int32_t)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&bufs.cur_mask), 2 * I));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&bufs.state), ST_STATE_WORDS * sizeof(int32_t)));
    st_cache *cache = st_cache_create(&bufs, I, H, ST_F32, 1);
    if (!cache) { std::printf("capi_client: st_cache_create: %s\n", st_last_error()); return 1; }
    ST_CALL(st_cache_load_weights(cache, d_gate, d_up, d_down, stream));   // nothing active yet

    // the worked trace of the reference: drop {1,3,5,7,9}, then add {1,3} and drop {0,2,4}
    std::vector<uint8_t> m1(I, 1), m2;
    for (int i : {1, 3, 5, 7, 9}) m1[i] = 0;
    m2 = m1;
    for (int i : {1, 3}) m2[i] = 1;
    for (int i : {0, 2, 4}) m2[i] = 0;
    const std::vector<int> want1 = {0, 15, 2, 14, 4, 13, 6, 12, 8, 11, 10};
    const std::vector<int> want2 = {1, 15, 3, 14, 10, 13, 6, 12, 8, 11};
    uint8_t *d_mask = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_mask), I));
    // the all-ones initial mask of the reference's constructor (weight_cache.h:226): order 0..I-1
    HIP_OK(hipMemset(d_mask, 1, I));
    ST_CALL(st_cache_update_async(cache, d_mask, stream));
    HIP_OK(hipStreamSynchronize(stream));
    const int64_t ws_bytes = st_mlp_workspace_bytes(1, H, I);
    void *d_ws = nullptr; float *d_out = nullptr, *d_comb = nullptr;
    HIP_OK(hipMalloc(&d_ws, ws_bytes)); HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_out), H * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_comb), 2 * I * sizeof(float)));

    auto check_step = [&](const std::vector<uint8_t> &mask, const std::vector<int> &want, bool fused) -> int {
        HIP_OK(hipMemcpy(d_mask, mask.data(), I, hipMemcpyHostToDevice));
        const int n = (int)want.size();
        if (fused) {
            ST_CALL(st_cache_update_forward(cache, d_mask, d_x, 1, n, d_out, d_comb, 2 * I, d_ws, ws_bytes, ST_ACT_SILU,
                                            stream));
        } else {
            ST_CALL(st_cache_update_async(cache, d_mask, stream));
            ST_CALL(st_mlp_forward(d_x, 1, H, bufs.gate_active, bufs.up_active, bufs.down_active, I,
                                   bufs.state + ST_STATE_N_ACTIVE, n, d_out, d_comb, 2 * I, d_ws, ws_bytes, ST_ACT_SILU,
                                   ST_F32, 1, stream));
        }
        int32_t state[ST_STATE_WORDS];
        ST_CALL(st_cache_sync_state(cache, state, stream));
        if (state[ST_STATE_N_ACTIVE] != n) { std::printf("capi_client: n_active %d, expected %d\n", state[ST_STATE_N_ACTIVE], n); return 1; }
        std::vector<int32_t> idx(2 * I);
        HIP_OK(hipMemcpy(idx.data(), bufs.indices, idx.size() * sizeof(int32_t), hipMemcpyDeviceToHost));
        const int32_t *cur = idx.data() + (size_t)state[ST_STATE_EPOCH] * I;
        for (int p = 0; p < n; ++p)
            if (cur[p] != want[p]) { std::printf("capi_client: position %d holds %d, expected %d\n", p, cur[p], want[p]); return 1; }
        // out = sum_j silu(<gate_j, x>) * <up_j, x> * down[:, j] over the active j
        std::vector<double> ref(H, 0.0);
        for (int j : want) {
            double g = 0, u = 0;
            for (int h = 0; h < H; ++h) { g += (double)gate[j * H + h] * x[h]; u += (double)up[j * H + h] * x[h]; }
            const double hv = silu((float)g) * u;
            for (int h = 0; h < H; ++h) ref[h] += hv * down[h * I + j];
        }
        std::vector<float> out(H);
        HIP_OK(hipMemcpy(out.data(), d_out, H * sizeof(float), hipMemcpyDeviceToHost));
        for (int h = 0; h < H; ++h)
            if (std::fabs(out[h] - ref[h]) > 1e-5 * (1.0 + std::fabs(ref[h]))) {
                std::printf("capi_client: out[%d] = %g, expected %g\n", h, out[h], ref[h]);
                return 1;
            }
        return 0;
    };
    if (check_step(m1, want1, false)) return 1;
    if (check_step(m2, want2, true)) return 1;

    // an update that would leave nothing active is reported, not applied
    std::vector<uint8_t> none(I, 0);
    HIP_OK(hipMemcpy(d_mask, none.data(), I, hipMemcpyHostToDevice));
    ST_CALL(st_cache_update_async(cache, d_mask, stream));
    if (st_cache_sync_state(cache, nullptr, stream) != ST_ERR_NO_ACTIVE) { std::printf("capi_client: empty mask not reported\n"); return 1; }

    // ---- predictor: mask[i] = (Bm (A x))[i] >= 0
    float *d_t = nullptr, *d_scores = nullptr; uint8_t *d_pm = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_t), r * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_scores), I * sizeof(float)));
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_pm), I));
    ST_CALL(st_predictor_mask(d_x, 1, H, d_A, r, d_Bm, I, ST_F32, 0.f, 1, d_t, d_scores, d_pm, stream));
    uint8_t *d_topk = nullptr;
    HIP_OK(hipMalloc(reinterpret_cast<void **>(&d_topk), I));
    ST_CALL(st_mask_select(d_scores, 1, I, ST_MASK_TOPK, 5, 0.f, d_topk, nullptr, nullptr, 0, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> scores(I); std::vector<uint8_t> pm(I), topk(I);
    HIP_OK(hipMemcpy(scores.data(), d_scores, I * sizeof(float), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(pm.data(), d_pm, I, hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(topk.data(), d_topk, I, hipMemcpyDeviceToHost));
    int selected = 0;
    for (int i = 0; i < I; ++i) {
        double t_ref[4] = {0, 0, 0, 0}, s = 0;
        for (int k = 0; k < r; ++k) { for (int h = 0; h < H; ++h) t_ref[k] += (double)A[k * H + h] * x[h]; s += t_ref[k] * Bm[i * r + k]; }
        if (std::fabs(scores[i] - s) > 1e-5) { std::printf("capi_client: score %d = %g, expected %g\n", i, scores[i], s); return 1; }
        if (pm[i] != (scores[i] >= 0.f ? 1 : 0)) { std::printf("capi_client: mask bit %d wrong\n", i); return 1; }
        int larger = 0;
        for (int j = 0; j < I; ++j) larger += scores[j] > scores[i] || (scores[j] == scores[i] && j < i);
        if (topk[i] != (larger < 5 ? 1 : 0)) { std::printf("capi_client: top-k bit %d wrong\n", i); return 1; }
        selected += topk[i];
    }
    if (selected != 5) { std::printf("capi_client: top-k selected %d\n", selected); return 1; }

    st_cache_destroy(cache);
    std::printf("capi_client: OK\n");
    return 0;
}
