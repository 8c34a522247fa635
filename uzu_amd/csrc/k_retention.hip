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

// ---- the chunk kernels on the matrix cores with f32 operands (v_mfma_f32_32x32x2_f32: products and sums in f32, nothing is rounded to bf16), head widths up
// to 128.  Lane l of a wave feeds A[row l % 32][k = l / 32] and B[k = l / 32][column l % 32]; its 16 results are rows 8 (r / 4) + 4 (l / 32) + r % 4 of column l % 32.
typedef float f32x16_m __attribute__((ext_vector_type(16)));

// A_c = (decayed keys)^T values: [dim][vdim] from 64 rows; tiles of 32 x 32 dealt round-robin to the four waves (at most four each)
__global__ void __launch_bounds__(256) retention_chunk_local_mfma_kernel(RetentionParams p, float* ws) {
    extern __shared__ float s_kv[]; // [64][KP] decayed keys, then [64][VP] values, zero-padded
    __shared__ float s_pw[kChunk + 1];
    uint32_t z, c;
    SeqSpan sp;
    if (!find_chunk(p, blockIdx.x, z, c, sp)) return;
    const uint32_t a = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5, dim = p.dim, vdim = p.vdim;
    const uint32_t TI = (dim + 31) / 32, TJ = (vdim + 31) / 32, KP = 32 * TI, VP = 32 * TJ;
    const uint32_t r0 = sp.row0 + c * kChunk, n = sp.count - c * kChunk < kChunk ? sp.count - c * kChunk : kChunk;
    if (tid == 0) {
        float w = 1.0f;
        const float decay = p.decay[a];
        for (uint32_t t = 0; t <= kChunk; ++t) s_pw[t] = w, w *= decay;
    }
    __syncthreads();
    float* s_k = s_kv;
    float* s_v = s_kv + (size_t)kChunk * KP;
    for (uint32_t e = tid; e < kChunk * KP; e += 256) {
        const uint32_t t = e / KP, i = e % KP;
        s_k[e] = (t < n && i < dim) ? p.qkv[(size_t)(r0 + t) * p.ld + p.k_col + a * dim + i] * s_pw[n - 1 - t] : 0.0f;
    }
    for (uint32_t e = tid; e < kChunk * VP; e += 256) {
        const uint32_t t = e / VP, j = e % VP;
        s_v[e] = (t < n && j < vdim) ? p.qkv[(size_t)(r0 + t) * p.ld + p.v_col + a * vdim + j] : 0.0f;
    }
    __syncthreads();
    f32x16_m acc[4];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[q][r] = 0.0f;
    const uint32_t tiles = TI * TJ, steps = (n + 1) / 2;
    for (uint32_t t2 = 0; t2 < steps; ++t2) {
        const uint32_t t = 2 * t2 + half;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t tt = wave + 4 * q;
            if (tt < tiles) acc[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_k[t * KP + (tt / TJ) * 32 + l32], s_v[t * VP + (tt % TJ) * 32 + l32], acc[q], 0, 0, 0);
        }
    }
    float* dst = ws + ((size_t)blockIdx.x * p.heads + a) * dim * vdim;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const uint32_t tt = wave + 4 * q;
        if (tt >= tiles) continue;
        const uint32_t j = (tt % TJ) * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t i = (tt / TJ) * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (i < dim && j < vdim) dst[(size_t)i * vdim + j] = acc[q][r];
        }
    }
}

// o_i = decay^(i+1) S_c^T q_i + sum_(j <= i) decay^(i-j) <q_i, k_j> v_j for the 64 rows of a chunk
__global__ void __launch_bounds__(256) retention_chunk_out_mfma_kernel(RetentionParams p, const float* ws) {
    constexpr uint32_t SW = 64, SP = SW + 1;        // a slab of 64 key coordinates, pitch 65: rows on distinct banks
    __shared__ float s_buf[2 * kChunk * SP];        // query slab + key slab; later the values [64][VP <= 128]
    __shared__ float s_p[kChunk][kChunk + 1], s_pw[kChunk + 2];
    uint32_t z, c;
    SeqSpan sp;
    if (!find_chunk(p, blockIdx.x, z, c, sp)) return;
    const uint32_t a = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, half = lane >> 5, dim = p.dim, vdim = p.vdim;
    const uint32_t TJ = (vdim + 31) / 32, VP = 32 * TJ;
    const uint32_t r0 = sp.row0 + c * kChunk, n = sp.count - c * kChunk < kChunk ? sp.count - c * kChunk : kChunk;
    if (tid == 0) {
        float w = 1.0f;
        const float decay = p.decay[a];
        for (uint32_t t = 0; t <= kChunk + 1; ++t) s_pw[t] = w, w *= decay;
    }
    const float* qb = p.qkv + (size_t)r0 * p.ld + p.q_col + a * dim;
    const float* kb = p.qkv + (size_t)r0 * p.ld + p.k_col + a * dim;
    const float* vb = p.qkv + (size_t)r0 * p.ld + p.v_col + a * vdim;
    float* s_q = s_buf;
    float* s_k = s_buf + kChunk * SP;
    // scores of the chunk's rows among themselves: wave w owns the 32 x 32 tile (w / 2, w % 2)
    const uint32_t pi = wave >> 1, pj = wave & 1;
    f32x16_m sc;
#pragma unroll
    for (int r = 0; r < 16; ++r) sc[r] = 0.0f;
    for (uint32_t d0 = 0; d0 < dim; d0 += SW) {
        __syncthreads();
        for (uint32_t e = tid; e < kChunk * SW; e += 256) {
            const uint32_t r = e / SW, dd = e % SW, d = d0 + dd;
            const bool ok = r < n && d < dim;
            s_q[r * SP + dd] = ok ? qb[(size_t)r * p.ld + d] : 0.0f;
            s_k[r * SP + dd] = ok ? kb[(size_t)r * p.ld + d] : 0.0f;
        }
        __syncthreads();
        const uint32_t dn = dim - d0 < SW ? dim - d0 : SW;
        for (uint32_t d = 0; d < dn; d += 2) sc = __builtin_amdgcn_mfma_f32_32x32x2f32(s_q[(pi * 32 + l32) * SP + d + half], s_k[(pj * 32 + l32) * SP + d + half], sc, 0, 0, 0);
    }
    __syncthreads(); // the slabs are done with, s_pw is there
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t i = pi * 32 + 8 * (r >> 2) + 4 * half + (r & 3), j = pj * 32 + l32;
        s_p[i][j] = (j <= i && i < n) ? sc[r] * s_pw[i - j] : 0.0f;
    }
    float* s_v = s_buf; // [64][VP]
    for (uint32_t e = tid; e < kChunk * VP; e += 256) {
        const uint32_t t = e / VP, j = e % VP;
        s_v[e] = (t < n && j < vdim) ? vb[(size_t)t * p.ld + j] : 0.0f;
    }
    __syncthreads();
    // outputs: tiles (row half oi, column tile oc), dealt round-robin to the waves (at most two each)
    const uint32_t tiles = 2 * TJ;
    f32x16_m o[2];
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[q][r] = 0.0f;
    const uint32_t steps = (n + 1) / 2;
    for (uint32_t j2 = 0; j2 < steps; ++j2) {
        const uint32_t j = 2 * j2 + half;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const uint32_t tt = wave + 4 * q;
            if (tt < tiles) o[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_p[(tt / TJ) * 32 + l32][j], s_v[j * VP + (tt % TJ) * 32 + l32], o[q], 0, 0, 0);
        }
    }
    if (sp.start || c) { // the carried state: + sum_d (decay^(i+1) q_i[d]) S[d][column], the state's rows straight from memory
        const float* S = ws + ((size_t)blockIdx.x * p.heads + a) * dim * vdim;
        for (uint32_t d0 = 0; d0 < dim; d0 += SW) {
            __syncthreads(); // the values (first slab) / the slab before have been read
            for (uint32_t e = tid; e < kChunk * SW; e += 256) {
                const uint32_t r = e / SW, dd = e % SW, d = d0 + dd;
                s_q[r * SP + dd] = (r < n && d < dim) ? qb[(size_t)r * p.ld + d] * s_pw[r + 1] : 0.0f;
            }
            __syncthreads();
            const uint32_t dn = dim - d0 < SW ? dim - d0 : SW;
            for (uint32_t d = 0; d < dn; d += 2) {
                const uint32_t dg = d0 + d + half;
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const uint32_t tt = wave + 4 * q;
                    if (tt >= tiles) continue;
                    const uint32_t col = (tt % TJ) * 32 + l32;
                    const float sv = (dg < dim && col < vdim) ? S[(size_t)dg * vdim + col] : 0.0f;
                    o[q] = __builtin_amdgcn_mfma_f32_32x32x2f32(s_q[((tt / TJ) * 32 + l32) * SP + d + half], sv, o[q], 0, 0, 0);
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const uint32_t tt = wave + 4 * q;
        if (tt >= tiles) continue;
        const uint32_t col = (tt % TJ) * 32 + l32;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t i = (tt / TJ) * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
            if (i < n && col < vdim) p.out[((size_t)(r0 + i) * p.heads + a) * vdim + col] = o[q][r];
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
    if (p.form == 2 || p.form == 3 || (p.form == 0 && p.chunk_ws && p.rows > 16 * p.nseq)) { // prompt-sized: in chunks (3: without the matrix cores)
        UZU_REQUIRE(p.chunk_ws && p.chunks && p.chunk_ws_bytes >= retention_chunk_ws_bytes(p.chunks, p.heads, p.dim, p.vdim), "retention: the chunked form needs its workspace");
        if (p.form != 3 && p.dim <= 128 && p.vdim <= 128) { // on the matrix cores with f32 operands
            const dim3 cgrid(p.chunks, p.heads);
            const size_t lds = (size_t)kChunk * (32 * ((p.dim + 31) / 32) + 32 * ((p.vdim + 31) / 32)) * 4;
            UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(retention_chunk_local_mfma_kernel, cgrid, dim3(256), lds, s, p, p.chunk_ws); }, "retention_chunk_local_mfma"));
            const dim3 sgrid(p.nseq, p.heads, std::min<uint32_t>((p.dim * p.vdim + 255) / 256, 1024));
            UZU_PROPAGATE(launch_check([&] { hipLaunchKernelGGL(retention_chunk_scan_kernel, sgrid, dim3(256), 0, s, p, p.chunk_ws); }, "retention_chunk_scan"));
            return launch_check([&] { hipLaunchKernelGGL(retention_chunk_out_mfma_kernel, cgrid, dim3(256), 0, s, p, (const float*)p.chunk_ws); }, "retention_chunk_out_mfma");
        }
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
