// k_retention.hip -- retention for the f32-stream designs (kernels_stream32.h): per head a decayed sum of outer products, S <- decay S + k v^T, read out as
// S^T q; no softmax, no denominator.  The state, the decays and every sum are f32.
//
// Token by token (this file's first kernel): a workgroup per (sequence, head) keeps the state in registers -- thread (j, part) owns S[i][j] for the rows
// i = part, part + parts, ... -- so the update and the thread's share of S^T q touch no memory; the shares of a column meet in LDS and are added in a fixed
// order.  The same kernel runs prompts and decode steps, so a prompt's state does not depend on how it was cut.
#include <algorithm>

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

// ---- in chunks of 64 rows (prompts).  With S_c the state in front of chunk c, n rows in the chunk and i, j its rows:
//   local      A_c = sum_j decay^(n-1-j) k_j v_j^T                                            (parallel over chunks)
//   scan       S_(c+1) = decay^n S_c + A_c, the sequence's state in front and behind          (chunk after chunk, element-wise)
//   out        o_i = decay^(i+1) S_c^T q_i + sum_(j <= i) decay^(i-j) <q_i, k_j> v_j            (parallel over chunks)
// Powers of the decay are formed by repeated multiplication (what the token-by-token form applies to its state).  ws holds one [dim][vdim] block per
// (chunk of the pass, head): first A_c, then S_c in its place.
constexpr uint32_t kChunk = 64;

__device__ __forceinline__ bool find_chunk(const RetentionParams& p, uint32_t index, uint32_t& z, uint32_t& c, SeqSpan& sp) {
    for (z = 0; z < p.nseq; ++z) {
        sp = p.spans[z];
        const uint32_t n = (sp.count + kChunk - 1) / kChunk;
        if (index < n) {
            c = index;
            return true;
        }
        index -= n;
    }
    return false;
}

template <int N>
__global__ void __launch_bounds__(256) retention_chunk_local_kernel(RetentionParams p, float* ws, uint32_t stage_rows) {
    extern __shared__ float s_kv[]; // [stage_rows][dim] keys, then [stage_rows][vdim] values
    uint32_t z, c;
    SeqSpan sp;
    if (!find_chunk(p, blockIdx.x, z, c, sp)) return;
    const uint32_t a = blockIdx.y, tid = threadIdx.x, dim = p.dim, vdim = p.vdim;
    const uint32_t parts = 256 / vdim, j = tid % vdim, part = tid / vdim;
    const bool active = part < parts;
    const uint32_t r0 = sp.row0 + c * kChunk, n = sp.count - c * kChunk < kChunk ? sp.count - c * kChunk : kChunk;
    const float decay = p.decay[a];
    float* s_k = s_kv;
    float* s_v = s_kv + (size_t)stage_rows * dim;
    float S[N];
#pragma unroll
    for (int q = 0; q < N; ++q) S[q] = 0.0f;
    for (uint32_t t0 = 0; t0 < n; t0 += stage_rows) {
        const uint32_t tn = n - t0 < stage_rows ? n - t0 : stage_rows;
        __syncthreads();
        for (uint32_t e = tid; e < tn * dim; e += 256) s_k[e] = p.qkv[(size_t)(r0 + t0 + e / dim) * p.ld + p.k_col + a * dim + e % dim];
        for (uint32_t e = tid; e < tn * vdim; e += 256) s_v[e] = p.qkv[(size_t)(r0 + t0 + e / vdim) * p.ld + p.v_col + a * vdim + e % vdim];
        __syncthreads();
        if (!active) continue;
        for (uint32_t t = 0; t < tn; ++t) {
            const float v = s_v[t * vdim + j];
#pragma unroll
            for (int q = 0; q < N; ++q) {
                const uint32_t i = part + q * parts;
                if (i < dim) S[q] = fmaf(decay, S[q], s_k[t * dim + i] * v);
            }
        }
    }
    float* dst = ws + ((size_t)blockIdx.x * p.heads + a) * dim * vdim;
#pragma unroll
    for (int q = 0; q < N; ++q) {
        const uint32_t i = part + q * parts;
        if (active && i < dim) dst[(size_t)i * vdim + j] = S[q];
    }
}

__global__ void __launch_bounds__(256) retention_chunk_scan_kernel(RetentionParams p, float* ws) {
    const uint32_t z = blockIdx.x, a = blockIdx.y;
    const SeqSpan sp = p.spans[z];
    if (!sp.count) return;
    uint32_t first = 0; // the sequence's first chunk among the pass's chunks
    for (uint32_t q = 0; q < z; ++q) first += (p.spans[q].count + kChunk - 1) / kChunk;
    const uint32_t chunks = (sp.count + kChunk - 1) / kChunk, elems = p.dim * p.vdim;
    const float decay = p.decay[a];
    float* state = p.states[z] + (size_t)a * elems;
    float pw_full = 1.0f;
    for (uint32_t t = 0; t < kChunk; ++t) pw_full *= decay;
    float pw_last = 1.0f;
    for (uint32_t t = 0; t < sp.count - (chunks - 1) * kChunk; ++t) pw_last *= decay;
    for (uint32_t e = blockIdx.z * 256 + threadIdx.x; e < elems; e += 256 * gridDim.z) { // the elements are independent of each other: one per thread
        float S = sp.start ? state[e] : 0.0f;
        for (uint32_t c = 0; c < chunks; ++c) {
            float* slot = ws + ((size_t)(first + c) * p.heads + a) * elems + e;
            const float local = *slot;
            *slot = S;
            S = fmaf(c + 1 == chunks ? pw_last : pw_full, S, local);
        }
        state[e] = S;
    }
}

// a thread owns rows 4 ty .. 4 ty + 3 (ty = tid / 16) and columns tx, tx + 16, ... (tx = tid % 16) of the chunk's scores and of its outputs
constexpr uint32_t kSlab = 32, kMaxCols = 16; // value widths up to 256
__global__ void __launch_bounds__(256) retention_chunk_out_kernel(RetentionParams p, const float* ws) {
    __shared__ float s_q[kChunk][kSlab + 1], s_k[kChunk][kSlab + 1], s_p[kChunk][kChunk + 1], s_pw[kChunk + 1];
    uint32_t z, c;
    SeqSpan sp;
    if (!find_chunk(p, blockIdx.x, z, c, sp)) return;
    const uint32_t a = blockIdx.y, tid = threadIdx.x, tx = tid & 15, ty = tid >> 4, dim = p.dim, vdim = p.vdim;
    const uint32_t r0 = sp.row0 + c * kChunk, n = sp.count - c * kChunk < kChunk ? sp.count - c * kChunk : kChunk;
    const float decay = p.decay[a];
    if (tid == 0) {
        float w = 1.0f;
        for (uint32_t t = 0; t <= kChunk; ++t) s_pw[t] = w, w *= decay;
    }
    const float* qb = p.qkv + (size_t)r0 * p.ld + p.q_col + a * dim;
    const float* kb = p.qkv + (size_t)r0 * p.ld + p.k_col + a * dim;
    const float* vb = p.qkv + (size_t)r0 * p.ld + p.v_col + a * vdim;
    float sc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) sc[i][j] = 0.0f;
    for (uint32_t d0 = 0; d0 < dim; d0 += kSlab) {
        __syncthreads();
        for (uint32_t e = tid; e < kChunk * kSlab; e += 256) {
            const uint32_t r = e / kSlab, d = d0 + e % kSlab;
            const bool ok = r < n && d < dim;
            s_q[r][e % kSlab] = ok ? qb[(size_t)r * p.ld + d] : 0.0f;
            s_k[r][e % kSlab] = ok ? kb[(size_t)r * p.ld + d] : 0.0f;
        }
        __syncthreads();
#pragma unroll 8
        for (uint32_t d = 0; d < kSlab; ++d) {
            float qa[4], ka[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) qa[i] = s_q[4 * ty + i][d], ka[i] = s_k[4 * tx + i][d];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) sc[i][j] = fmaf(qa[i], ka[j], sc[i][j]);
        }
    }
    __syncthreads(); // s_pw is there, the slabs are done with
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t r = 4 * ty + i, col = 4 * tx + j;
            s_p[r][col] = (col <= r && r < n) ? sc[i][j] * s_pw[r - col] : 0.0f;
        }
    __syncthreads();
    float o[4][kMaxCols];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (uint32_t m = 0; m < kMaxCols; ++m) o[i][m] = 0.0f;
    // the carried state: o_i += sum_d (decay^(i+1) q_i[d]) S[d][col]
    if (sp.start || c) {
        const float* S = ws + ((size_t)blockIdx.x * p.heads + a) * dim * vdim;
        float wq[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) wq[i] = s_pw[4 * ty + i + 1];
        for (uint32_t d = 0; d < dim; ++d) {
            float qa[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) qa[i] = 4 * ty + i < n ? qb[(size_t)(4 * ty + i) * p.ld + d] * wq[i] : 0.0f;
#pragma unroll
            for (uint32_t m = 0; m < kMaxCols; ++m) {
                const uint32_t col = tx + 16 * m;
                if (col >= vdim) break;
                const float sv = S[(size_t)d * vdim + col];
#pragma unroll
                for (int i = 0; i < 4; ++i) o[i][m] = fmaf(qa[i], sv, o[i][m]);
            }
        }
    }
    // the chunk's own rows: o_i += sum_(j <= i) P[i][j] v_j[col]
    const uint32_t jmax = 4 * ty + 3 < n ? 4 * ty + 3 : n - 1;
    for (uint32_t j = 0; j <= jmax; ++j) {
        float pa[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) pa[i] = s_p[4 * ty + i][j];
#pragma unroll
        for (uint32_t m = 0; m < kMaxCols; ++m) {
            const uint32_t col = tx + 16 * m;
            if (col >= vdim) break;
            const float v = vb[(size_t)j * p.ld + col];
#pragma unroll
            for (int i = 0; i < 4; ++i) o[i][m] = fmaf(pa[i], v, o[i][m]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t r = 4 * ty + i;
        if (r >= n) continue;
#pragma unroll
        for (uint32_t m = 0; m < kMaxCols; ++m) {
            const uint32_t col = tx + 16 * m;
            if (col >= vdim) break;
            p.out[((size_t)(r0 + r) * p.heads + a) * vdim + col] = o[i][m];
        }
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

size_t retention_chunk_ws_bytes(uint32_t chunks, uint32_t heads, uint32_t dim, uint32_t vdim) { return (size_t)chunks * heads * dim * vdim * 4; }

bool retention_supported(uint32_t dim, uint32_t vdim) { return dim && vdim && vdim <= 256 && dim <= 512 && (dim + (256 / vdim) - 1) / (256 / vdim) <= 128; }

uzu_status retention(hipStream_t s, const RetentionParams& p) {
    if (!p.rows || !p.nseq) return UZU_OK;
    UZU_REQUIRE(p.qkv && p.out && p.states && p.decay && p.spans && p.heads, "retention: null argument");
    UZU_UNSUPPORTED(!retention_supported(p.dim, p.vdim), "retention: head widths %u x %u (keys up to 512, values up to 256)", p.dim, p.vdim);
    UZU_REQUIRE(p.heads <= 65535, "retention: too many heads for one launch");
    const uint32_t parts = 256 / p.vdim, per = (p.dim + parts - 1) / parts;
    const dim3 grid(p.nseq, p.heads);
    if (p.form == 2 || (p.form == 0 && p.chunk_ws && p.rows > 16 * p.nseq)) { // prompt-sized: in chunks
        UZU_REQUIRE(p.chunk_ws && p.chunks && p.chunk_ws_bytes >= retention_chunk_ws_bytes(p.chunks, p.heads, p.dim, p.vdim), "retention: the chunked form needs its workspace");
        uint32_t stage = 16384 / (p.dim + p.vdim);
        stage = stage >= 64 ? 64 : stage >= 32 ? 32 : stage >= 16 ? 16 : 8;
        const dim3 cgrid(p.chunks, p.heads);
        const size_t lds = (size_t)stage * (p.dim + p.vdim) * 4;
#define UZU_LOC(N) UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(retention_chunk_local_kernel<N>, cgrid, dim3(256), lds, s, p, p.chunk_ws, stage); }, "retention_chunk_local"))
        if (per <= 8) UZU_LOC(8);
        else if (per <= 16) UZU_LOC(16);
        else if (per <= 32) UZU_LOC(32);
        else if (per <= 64) UZU_LOC(64);
        else UZU_LOC(128);
#undef UZU_LOC
        const dim3 sgrid(p.nseq, p.heads, std::min<uint32_t>((p.dim * p.vdim + 255) / 256, 1024));
        UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(retention_chunk_scan_kernel, sgrid, dim3(256), 0, s, p, p.chunk_ws); }, "retention_chunk_scan"));
        return launch_check([&] { hipLaunchKernelGGL(retention_chunk_out_kernel, cgrid, dim3(256), 0, s, p, (const float*)p.chunk_ws); }, "retention_chunk_out");
    }
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
