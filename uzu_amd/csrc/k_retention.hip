// k_retention.hip -- retention for the f32-stream designs (kernels_stream32.h): per head a decayed sum of outer products, S <- decay S + k v^T, read out as
// S^T q; no softmax, no denominator.  The state, the decays and every sum are f32.
//
// Token by token (this file's first kernel): a workgroup per (sequence, head) keeps the state in registers -- thread (j, part) owns S[i][j] for the rows
// i = part, part + parts, ... -- so the update and the thread's share of S^T q touch no memory; the shares of a column meet in LDS and are added in a fixed
// order.  The same kernel runs prompts and decode steps, so a prompt's state does not depend on how it was cut.
#include "device_utils.h"
#include "kernels_stream32.h"

namespace uzu {
namespace k {

namespace {

template <int N> // state elements per thread
__global__ void __launch_bounds__(256) retention_steps_kernel(RetentionParams p) {
    __shared__ float s_q[512], s_k[512], s_v[256], s_part[256];
    const uint32_t z = blockIdx.x, a = blockIdx.y, tid = threadIdx.x;
    const SeqSpan sp = p.spans[z];
    if (!sp.count) return;
    const uint32_t dim = p.dim, vdim = p.vdim;
    const uint32_t parts = 256 / vdim, j = tid % vdim, part = tid / vdim;
    const bool active = part < parts;
    float* state = p.states[z] + (size_t)a * dim * vdim;
    const float decay = p.decay[a];
    float S[N];
#pragma unroll
    for (int n = 0; n < N; ++n) {
        const uint32_t i = part + n * parts;
        S[n] = (active && i < dim && sp.start) ? state[(size_t)i * vdim + j] : 0.0f;
    }
    for (uint32_t step = 0; step < sp.count; ++step) {
        const float* row = p.qkv + (size_t)(sp.row0 + step) * p.ld;
        for (uint32_t c = tid; c < dim; c += 256) s_q[c] = row[p.q_col + a * dim + c], s_k[c] = row[p.k_col + a * dim + c];
        if (tid < vdim) s_v[tid] = row[p.v_col + a * vdim + tid];
        __syncthreads();
        float sum = 0.0f;
        if (active) {
            const float v = s_v[j];
#pragma unroll
            for (int n = 0; n < N; ++n) {
                const uint32_t i = part + n * parts;
                if (i < dim) {
                    S[n] = fmaf(decay, S[n], s_k[i] * v);
                    sum = fmaf(S[n], s_q[i], sum);
                }
            }
        }
        s_part[tid] = sum;
        __syncthreads();
        if (tid < vdim) {
            float total = s_part[tid];
            for (uint32_t q = 1; q < parts; ++q) total += s_part[q * vdim + tid];
            p.out[((size_t)(sp.row0 + step) * p.heads + a) * vdim + tid] = total;
        }
        __syncthreads();
    }
#pragma unroll
    for (int n = 0; n < N; ++n) {
        const uint32_t i = part + n * parts;
        if (active && i < dim) state[(size_t)i * vdim + j] = S[n];
    }
}

// a wave per (row, head)
__global__ void __launch_bounds__(64) head_rms_gate_kernel(float* x, const float* gate, uint32_t ldg, float eps, uint32_t heads, uint32_t width) {
    const uint32_t r = blockIdx.x, a = blockIdx.y, lane = threadIdx.x;
    float* h = x + ((size_t)r * heads + a) * width;
    float acc = 0.0f;
    for (uint32_t c = lane; c < width; c += 64) acc = fmaf(h[c], h[c], acc);
    const float inv = 1.0f / sqrtf(wave_sum(acc) / (float)width + eps);
    for (uint32_t c = lane; c < width; c += 64) {
        float v = h[c] * inv;
        if (gate) {
            const float g = gate[(size_t)r * ldg + (size_t)a * width + c];
            v *= g / (1.0f + expf(-g));
        }
        h[c] = v;
    }
}

} // namespace

bool retention_supported(uint32_t dim, uint32_t vdim) { return dim && vdim && vdim <= 256 && dim <= 512 && (dim + (256 / vdim) - 1) / (256 / vdim) <= 128; }

uzu_status retention_chunked(hipStream_t s, const RetentionParams& p); // below, once it exists

uzu_status retention(hipStream_t s, const RetentionParams& p) {
    if (!p.rows || !p.nseq) return UZU_OK;
    UZU_REQUIRE(p.qkv && p.out && p.states && p.decay && p.spans && p.heads, "retention: null argument");
    UZU_UNSUPPORTED(!retention_supported(p.dim, p.vdim), "retention: head widths %u x %u (keys up to 512, values up to 256)", p.dim, p.vdim);
    UZU_REQUIRE(p.heads <= 65535, "retention: too many heads for one launch");
    const uint32_t parts = 256 / p.vdim, per = (p.dim + parts - 1) / parts;
    const dim3 grid(p.nseq, p.heads);
#define UZU_RET(N) return launch_check([&] { hipLaunchKernelGGL(retention_steps_kernel<N>, grid, dim3(256), 0, s, p); }, "retention")
    if (per <= 8) UZU_RET(8);
    if (per <= 16) UZU_RET(16);
    if (per <= 32) UZU_RET(32);
    if (per <= 64) UZU_RET(64);
    UZU_RET(128);
#undef UZU_RET
}

uzu_status head_rms_gate(hipStream_t s, float* x, const float* gate, uint32_t ldg, float eps, uint32_t rows, uint32_t heads, uint32_t width) {
    if (!rows || !heads) return UZU_OK;
    UZU_REQUIRE(x && width && heads <= 65535, "head_rms_gate: null argument");
    return launch_check([&] { hipLaunchKernelGGL(head_rms_gate_kernel, dim3(rows, heads), dim3(64), 0, s, x, gate, ldg, eps, heads, width); }, "head_rms_gate");
}

} // namespace k
} // namespace uzu
