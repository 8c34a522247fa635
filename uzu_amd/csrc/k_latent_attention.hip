// k_latent_attention.hip -- attention over a cached low-rank latent (UZU_MIXER_LATENT_ATTENTION; kernels_stream32.h).
//
// Per token the state keeps ONE row c = RMSNorm(W_down h) of `rank` numbers for all heads.  A head's key is W_up_k c and its value W_up_v c, so
//   score(i, j) = <q_i, W_up_k c_j> = <W_up_k^T q_i, c_j>          and          sum_j p_j W_up_v c_j = W_up_v (sum_j p_j c_j):
// the engine folds W_up_k into the query (a batched product per head) and applies W_up_v to the result, and the core below is attention with one shared
// "key = value" row per token in latent space -- the cache is read once per (row, head) and never expanded.  Scores, the softmax and the weighted sum are f32
// in both precisions; a sink adds exp(sink_h) to the denominator and nothing to the sum; the window keeps keys t - window < j <= t.
//
// The summation order over the keys depends on the row's position and the window only, so a row's result is the same whatever else the pass carries.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

__device__ __forceinline__ float cache_ld(const void* c, uint32_t bf16, size_t i) { return bf16 ? bf16_to_f32(((const uint16_t*)c)[i]) : ((const float*)c)[i]; }

// a wave per row
__global__ void __launch_bounds__(256) latent_norm_append_kernel(const float* x, const float* scales, float eps, void* const* caches, uint32_t cache_bf16, const SeqSpan* spans,
                                                                 const uint32_t* row_seq, uint32_t rows, uint32_t rank) {
    const uint32_t lane = threadIdx.x & 63, r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float* xr = x + (size_t)r * rank;
    float ss = 0.0f;
    for (uint32_t i = lane; i < rank; i += 64) ss = fmaf(xr[i], xr[i], ss);
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
    const uint32_t q = row_seq[r];
    const SeqSpan sp = spans[q];
    const size_t base = (size_t)(sp.start + (r - sp.row0)) * rank;
    void* c = caches[q];
    for (uint32_t i = lane; i < rank; i += 64) {
        const float v = xr[i] * inv * scales[i];
        if (cache_bf16) ((uint16_t*)c)[base + i] = f32_to_bf16(v);
        else ((float*)c)[base + i] = v;
    }
}

// Simple form: a wave per (row, head), lane = latent elements lane, lane + 64, ...; the keys one after the other with a running maximum.
template <int NT>
__global__ void __launch_bounds__(256) latent_attention_rows_kernel(LatentAttentionParams p) {
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t item = blockIdx.x * 4 + (threadIdx.x >> 6); // (row, head), heads of a row next to each other: they read the same latents
    if (item >= p.rows * p.heads) return;
    const uint32_t r = item / p.heads, h = item % p.heads;
    const uint32_t q = p.row_seq[r];
    const SeqSpan sp = p.spans[q];
    const uint32_t t = sp.start + (r - sp.row0);
    const uint32_t lo = (p.window && t + 1 > p.window) ? t + 1 - p.window : 0;
    const void* cache = p.caches[q];
    const float* ql = p.qlat + ((size_t)r * p.heads + h) * p.rank;
    float qv[NT], acc[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const uint32_t e = i * 64 + lane;
        qv[i] = e < p.rank ? ql[e] * p.scale : 0.0f;
        acc[i] = 0.0f;
    }
    // the sink takes part in the maximum and in the denominator only
    float m = p.sinks ? p.sinks[h] : -INFINITY;
    float l = p.sinks ? 1.0f : 0.0f;
    for (uint32_t j = lo; j <= t; ++j) {
        float cv[NT];
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            const uint32_t e = i * 64 + lane;
            cv[i] = e < p.rank ? cache_ld(cache, p.cache_bf16, (size_t)j * p.rank + e) : 0.0f;
            s = fmaf(qv[i], cv[i], s);
        }
        s = wave_sum(s);
        const float mn = fmaxf(m, s);
        const float corr = expf(m - mn), pj = expf(s - mn); // m == -inf only before the first key of a sink-less head: corr = 0 on l = 0
        l = fmaf(l, corr, pj);
#pragma unroll
        for (int i = 0; i < NT; ++i) acc[i] = fmaf(acc[i], corr, pj * cv[i]);
        m = mn;
    }
    const float inv = 1.0f / l;
    float* out = p.out + ((size_t)r * p.heads + h) * p.rank;
#pragma unroll
    for (int i = 0; i < NT; ++i) {
        const uint32_t e = i * 64 + lane;
        if (e < p.rank) out[e] = acc[i] * inv;
    }
}

} // namespace

uzu_status latent_norm_append(hipStream_t s, const float* x, const float* scales, float eps, void* const* caches, uint32_t cache_bf16, const SeqSpan* spans,
                              const uint32_t* row_seq, uint32_t rows, uint32_t rank) {
    if (!rows) return UZU_OK;
    UZU_REQUIRE(x && scales && caches && spans && row_seq && rank, "latent_norm_append: null argument");
    return launch_check([&] { hipLaunchKernelGGL(latent_norm_append_kernel, dim3((rows + 3) / 4), dim3(256), 0, s, x, scales, eps, caches, cache_bf16, spans, row_seq, rows, rank); },
                        "latent_norm_append");
}

uzu_status latent_attention(hipStream_t s, const LatentAttentionParams& p) {
    if (!p.rows) return UZU_OK;
    UZU_REQUIRE(p.qlat && p.out && p.caches && p.spans && p.row_seq && p.heads && p.rank, "latent_attention: null argument");
    UZU_UNSUPPORTED(p.rank > kLatentMaxRank, "latent_attention: latent rank %u above %u", p.rank, kLatentMaxRank);
    const uint32_t items = p.rows * p.heads;
    const dim3 grid((items + 3) / 4), block(256);
    const uint32_t nt = (p.rank + 63) / 64;
    if (nt <= 1) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<1>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 2) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<2>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 4) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<4>, grid, block, 0, s, p); }, "latent_attention");
    if (nt <= 8) return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<8>, grid, block, 0, s, p); }, "latent_attention");
    return launch_check([&] { hipLaunchKernelGGL(latent_attention_rows_kernel<16>, grid, block, 0, s, p); }, "latent_attention");
}

} // namespace k
} // namespace uzu
