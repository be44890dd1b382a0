// The gated delta rule with one decay per key channel, for gfx950.
//
// Per head, with S [key channel, value channel] float32 carried from token to token:
//     S <- diag(g_t) S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
// Four kernels:
//   delta_prepare      per token, in parallel: the short causal convolutions of q, k, v with silu, the unit
//                      norms of q and k, beta = sigmoid, g = exp(-exp(A) softplus(z + dt)), the output gate
//   conv_state_update  per sequence: the last taps - 1 inputs of the convolutions, kept for the next step
//   delta_rule         per (sequence, head, group of value channels): the recurrence over the step's tokens
//   headnorm_gate      o / rms(o) * w * gate per head, rounded to the compute type for the output product
//
// The columns of S are independent of one another: u_t[j] and o_t[j] need column j alone.  A column is
// held by PARTS neighbouring lanes, KPT key channels each, in registers for the whole step; the three
// dot products of a token (S^T k, S^T q, k . q) are finished with PARTS-wide butterflies, and one pass
// over the registers serves both the decay and the dot products, because
//     o_t = (gS)^T q + u_t (k . q).
// The state is stored transposed, [head, value channel, key channel], so that the lanes of a column
// read and write neighbouring pieces.  Compiled per (KPT, PARTS); the key size is KPT * PARTS.
#include "common.h"

#include <algorithm>

#ifndef KPT
#define KPT 4
#endif
#ifndef PARTS
#define PARTS 16
#endif

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z * sigmoid_f(z); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// proj float32 [T, proj_cols]: q [G*dk] | k [G*dk] | v [H*dv] | b [H] as projected.
// low float32 [T, H*dk + H*dv]: the decay's pre-activation, then the output gate's.
// conv float32 [C, taps] with C = 2*G*dk + H*dv (the filters of q, k, v stacked).
// state float32 [slots, state_stride]; the convolutions' inputs lie at conv_off as [taps - 1, C].
// prep float32 [T, prep_cols]: q | k | v | beta [H] | g [H*dk] | gate [H*dv].
__global__ void delta_prepare_kernel(const float* __restrict__ proj, const float* __restrict__ low,
                                     const float* __restrict__ conv, const float* __restrict__ a_log,
                                     const float* __restrict__ dt_bias, const float* __restrict__ state,
                                     const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
                                     const int32_t* __restrict__ state_slot, float* __restrict__ prep,
                                     int G, int H, int dk, int dv, int taps, int proj_cols, size_t state_stride,
                                     size_t conv_off) {
    extern __shared__ float qk[];              // q then k after convolution and silu: 2 * G * dk
    const int t = blockIdx.x;
    const int s = seq_of_token[t];
    const int i = t - q_start[s];              // place of the token in its portion
    const int QK = 2 * G * dk, C = QK + H * dv;
    const int prep_cols = C + H + H * dk + H * dv;
    const float* hist = state + static_cast<size_t>(state_slot[s]) * state_stride + conv_off;
    float* out = prep + static_cast<size_t>(t) * prep_cols;
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float acc = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int back = taps - 1 - j;
            const float x = (i - back >= 0) ? proj[static_cast<size_t>(t - back) * proj_cols + c]
                                            : hist[static_cast<size_t>(taps - 1 + i - back) * C + c];
            acc += conv[static_cast<size_t>(c) * taps + j] * x;
        }
        const float y = silu_f(acc);
        if (c < QK) qk[c] = y; else out[c] = y;
    }
    // beta, decay, gate
    const float* prow = proj + static_cast<size_t>(t) * proj_cols;
    const float* lrow = low + static_cast<size_t>(t) * (H * dk + H * dv);
    for (int c = threadIdx.x; c < H; c += blockDim.x) out[C + c] = sigmoid_f(prow[C + c]);
    for (int c = threadIdx.x; c < H * dk; c += blockDim.x)
        out[C + H + c] = expf(-expf(a_log[c / dk]) * softplus_f(lrow[c] + dt_bias[c]));
    for (int c = threadIdx.x; c < H * dv; c += blockDim.x) out[C + H + H * dk + c] = sigmoid_f(lrow[H * dk + c]);
    __syncthreads();
    // unit vectors per head of q and of k; q also times dk^(-1/2)
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
    const float qscale = 1.0f / sqrtf(static_cast<float>(dk));
    for (int head = wave; head < 2 * G; head += waves) {
        const float* v = qk + head * dk;
        float ss = 0.f;
        for (int c = lane; c < dk; c += WAVE) ss += v[c] * v[c];
        ss = wave_sum(ss);
        const float inv = (1.0f / sqrtf(ss + 1e-6f)) * (head < G ? qscale : 1.0f);
        for (int c = lane; c < dk; c += WAVE) out[head * dk + c] = v[c] * inv;
    }
}

__global__ void conv_state_update_kernel(const float* __restrict__ proj, float* __restrict__ state,
                                         const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                         const int32_t* __restrict__ state_slot, int C, int taps, int proj_cols,
                                         size_t state_stride, size_t conv_off) {
    const int s = blockIdx.x;
    const int n = q_len[s], first = q_start[s];
    float* hist = state + static_cast<size_t>(state_slot[s]) * state_stride + conv_off;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        // ascending j: entry j + n is read before any entry at or beyond it is written
        for (int j = 0; j < taps - 1; ++j) {
            const int i = n - (taps - 1) + j;
            hist[static_cast<size_t>(j) * C + c] = i >= 0 ? proj[static_cast<size_t>(first + i) * proj_cols + c]
                                                           : hist[static_cast<size_t>(j + n) * C + c];
        }
    }
}

// One workgroup: COLS = 256 / PARTS value channels of one head of one sequence.
__global__ void __launch_bounds__(256)
delta_rule_kernel(const float* __restrict__ prep, float* __restrict__ state, const int32_t* __restrict__ q_start,
                  const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot, float* __restrict__ o,
                  int G, int H, int dv, size_t state_stride) {
    constexpr int DK = KPT * PARTS, COLS = 256 / PARTS;
    const int s = blockIdx.x, h = blockIdx.y;
    const int part = threadIdx.x % PARTS;
    const int col = blockIdx.z * COLS + threadIdx.x / PARTS;
    const bool live = col < dv;
    const int g = h / (H / G);
    const int QK = 2 * G * DK, C = QK + H * dv;
    const int prep_cols = C + H + H * DK + H * dv;
    const int n = q_len[s];
    const float* row = prep + static_cast<size_t>(q_start[s]) * prep_cols;
    float* S_mem = state + static_cast<size_t>(state_slot[s]) * state_stride +
                   (static_cast<size_t>(h) * dv + (live ? col : 0)) * DK + part * KPT;
    float S[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) S[i] = live ? S_mem[i] : 0.f;
    const int q_at = g * DK + part * KPT, k_at = G * DK + g * DK + part * KPT;
    const int v_at = QK + h * dv + (live ? col : 0), b_at = C + h, g_at = C + H + h * DK + part * KPT;
    float q[KPT], k[KPT], dec[KPT], v, beta;
#pragma unroll
    for (int i = 0; i < KPT; ++i) { q[i] = row[q_at + i]; k[i] = row[k_at + i]; dec[i] = row[g_at + i]; }
    v = row[v_at];
    beta = row[b_at];
    for (int t = 0; t < n; ++t) {
        // the next token's operands are asked for before this token's arithmetic
        float qn[KPT], kn[KPT], dn[KPT], vn = 0.f, bn = 0.f;
        const bool more = t + 1 < n;
        const float* next = row + prep_cols;
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            qn[i] = more ? next[q_at + i] : 0.f;
            kn[i] = more ? next[k_at + i] : 0.f;
            dn[i] = more ? next[g_at + i] : 0.f;
        }
        if (more) { vn = next[v_at]; bn = next[b_at]; }
        float a = 0.f, b = 0.f, kq = 0.f;
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            S[i] *= dec[i];
            a += S[i] * k[i];
            b += S[i] * q[i];
            kq += k[i] * q[i];
        }
#pragma unroll
        for (int off = 1; off < PARTS; off <<= 1) {
            a += __shfl_xor(a, off, WAVE);
            b += __shfl_xor(b, off, WAVE);
            kq += __shfl_xor(kq, off, WAVE);
        }
        const float u = beta * (v - a);
#pragma unroll
        for (int i = 0; i < KPT; ++i) S[i] += k[i] * u;
        if (live && part == 0) o[(static_cast<size_t>(q_start[s]) + t) * (H * dv) + h * dv + col] = b + u * kq;
#pragma unroll
        for (int i = 0; i < KPT; ++i) { q[i] = qn[i]; k[i] = kn[i]; dec[i] = dn[i]; }
        v = vn;
        beta = bn;
        row = next;
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) S_mem[i] = S[i];
    }
}

// y[t, h, :] = o[t, h, :] / sqrt(mean(o[t, h, :]^2) + eps) * w * gate[t, h, :]; one wavefront a (token, head)
template <typename T>
__global__ void headnorm_gate_kernel(const float* __restrict__ o, const float* __restrict__ gate, size_t gate_stride,
                                     const float* __restrict__ w, T* __restrict__ y, int rows, int H, int dv, float eps) {
    const int lane = threadIdx.x & (WAVE - 1);
    const int r = blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;      // t * H + h
    if (r >= rows) return;
    const int t = r / H, h = r % H;
    const float* orow = o + static_cast<size_t>(r) * dv;
    const float* grow = gate + static_cast<size_t>(t) * gate_stride + h * dv;
    float ss = 0.f;
    for (int c = lane; c < dv; c += WAVE) ss += orow[c] * orow[c];
    ss = wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(dv) + eps);
    for (int c = lane; c < dv; c += WAVE) st(y + static_cast<size_t>(r) * dv + c, ((orow[c] * inv) * w[c]) * grow[c]);
}

NI_EXPORT int ni_delta_key_size() { return KPT * PARTS; }

NI_EXPORT int ni_delta_prepare(const void* proj, const void* low, const void* conv, const void* a_log, const void* dt_bias,
                               void* state, const void* seq_of_token, const void* q_start, const void* q_len,
                               const void* state_slot, void* prep, int T, int B, int G, int H, int dk, int dv, int taps,
                               int proj_cols, size_t state_stride, size_t conv_off, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dk != KPT * PARTS) return -1;
    const int C = 2 * G * dk + H * dv;
    const size_t lds = static_cast<size_t>(2 * G * dk) * sizeof(float);
    if (lds > 64 * 1024) return -2;
    delta_prepare_kernel<<<T, 256, lds, stream>>>((const float*)proj, (const float*)low, (const float*)conv,
                                                  (const float*)a_log, (const float*)dt_bias, (const float*)state,
                                                  (const int32_t*)seq_of_token, (const int32_t*)q_start,
                                                  (const int32_t*)state_slot, (float*)prep, G, H, dk, dv, taps, proj_cols,
                                                  state_stride, conv_off);
    if (taps > 1) {
        dim3 grid(B, std::max(1, std::min(64, (C + 255) / 256)));
        conv_state_update_kernel<<<grid, 256, 0, stream>>>((const float*)proj, (float*)state, (const int32_t*)q_start,
                                                           (const int32_t*)q_len, (const int32_t*)state_slot, C, taps,
                                                           proj_cols, state_stride, conv_off);
    }
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_delta_rule(const void* prep, void* state, const void* q_start, const void* q_len, const void* state_slot,
                            void* o, const void* norm_w, void* y, int T, int B, int G, int H, int dk, int dv, float eps,
                            size_t state_stride, int dtype, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (dk != KPT * PARTS) return -1;
    constexpr int COLS = 256 / PARTS;
    dim3 grid(B, H, (dv + COLS - 1) / COLS);
    delta_rule_kernel<<<grid, 256, 0, stream>>>((const float*)prep, (float*)state, (const int32_t*)q_start,
                                                (const int32_t*)q_len, (const int32_t*)state_slot, (float*)o, G, H, dv,
                                                state_stride);
    const int C = 2 * G * dk + H * dv;
    const int prep_cols = C + H + H * dk + H * dv;
    const float* gate = (const float*)prep + C + H + H * dk;
    const int rows = T * H;
    if (dtype == 0)
        headnorm_gate_kernel<float><<<(rows + 3) / 4, 256, 0, stream>>>((const float*)o, gate, prep_cols, (const float*)norm_w,
                                                                        (float*)y, rows, H, dv, eps);
    else
        headnorm_gate_kernel<bf16_t><<<(rows + 3) / 4, 256, 0, stream>>>((const float*)o, gate, prep_cols, (const float*)norm_w,
                                                                         (bf16_t*)y, rows, H, dv, eps);
    return NI_LAUNCH_RESULT();
}
