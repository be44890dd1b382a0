// Mixers whose memory of the past is a state of fixed size per request, for gfx950: linear attention with one
// decay a head, and the selective scan (a diagonal recurrence per channel whose step sizes, inputs and read-outs
// depend on the token) with its short causal convolution.
//
// Everything that enters a recurrence is float32: the projections come as float32 rows, states live in float32 in
// the cache manager's state slots, exponentials and softplus are the accurate routines.  A step brings, for every
// sequence b, the rows q_start[b] .. q_start[b] + q_len[b] - 1 (consecutive tokens of that sequence) and the slot
// state_slot[b]; a kernel walks a sequence's rows in order and leaves the state as it is after the last one.
// Every entry point returns 0 or a hipError_t.
#include "common.h"

#include <algorithm>

static inline unsigned blocks_of(size_t n, unsigned per) { return static_cast<unsigned>((n + per - 1) / per); }

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// sum over `parts` neighbouring lanes (a power of two), every one of them gets it
__device__ __forceinline__ float parts_sum(float v, int parts) {
    for (int off = 1; off < parts; off <<= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

// ---------------------------------------------------------------- silu of the first n columns of every row
__global__ void silu_rows_kernel(const float* __restrict__ in, int in_stride, float* __restrict__ out, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t t = i / n;
    const int c = static_cast<int>(i % n);
    out[i] = silu_f(in[t * in_stride + c]);
}

NI_EXPORT int ni_silu_rows(const void* in, int in_stride, void* out, int T, int n, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * n;
    if (total == 0) return 0;
    if (in_stride < n) return -1;
    silu_rows_kernel<<<blocks_of(total, 256), 256, 0, stream>>>((const float*)in, in_stride, (float*)out, n, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- linear attention with a decay a head
//   S <- decay[h] S + k v^T,   o = S^T q          S [dk, dv] per head, float32
// act float32 [T, 2 H dk + H dv]: q | k | v (after their activation), head by head.  The state of a slot is
// [H][dv][dkp] (a value channel's column of key channels lies together), dkp = parts * 8 >= dk, the padding zero.
// A column is held by `parts` neighbouring lanes with eight key channels each; a wavefront takes 64 / parts
// columns, a workgroup of four wavefronts four times that.  The next token's operands are asked for before this
// token's arithmetic.
#define DKPT 8

struct DecayOperands {
    float q[DKPT], k[DKPT], v;
};

__device__ __forceinline__ void decay_load(DecayOperands& o, const float* __restrict__ row, int q_off, int k_off, int v_off,
                                           int ch, int dk, bool whole) {
    if (whole) {
        const float4 a = *reinterpret_cast<const float4*>(row + q_off + ch), b = *reinterpret_cast<const float4*>(row + q_off + ch + 4);
        const float4 c = *reinterpret_cast<const float4*>(row + k_off + ch), d = *reinterpret_cast<const float4*>(row + k_off + ch + 4);
        o.q[0] = a.x; o.q[1] = a.y; o.q[2] = a.z; o.q[3] = a.w; o.q[4] = b.x; o.q[5] = b.y; o.q[6] = b.z; o.q[7] = b.w;
        o.k[0] = c.x; o.k[1] = c.y; o.k[2] = c.z; o.k[3] = c.w; o.k[4] = d.x; o.k[5] = d.y; o.k[6] = d.z; o.k[7] = d.w;
    } else {
#pragma unroll
        for (int i = 0; i < DKPT; ++i) {
            const bool in = ch + i < dk;
            o.q[i] = in ? row[q_off + ch + i] : 0.f;
            o.k[i] = in ? row[k_off + ch + i] : 0.f;
        }
    }
    o.v = row[v_off];
}

__global__ void __launch_bounds__(256)
decay_attention_kernel(const float* __restrict__ act, int act_stride, const float* __restrict__ decay, float* __restrict__ state,
                       size_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                       const int32_t* __restrict__ state_slot, float* __restrict__ out, int H, int dk, int dv, int parts) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int cols = WAVE / parts;
    const int part = lane % parts;
    const int c = (blockIdx.x * (blockDim.x / WAVE) + wave) * cols + lane / parts;
    const int n = q_len[b];
    if (c >= dv || n <= 0) return;               // whole groups of `parts` lanes leave together
    const int dkp = parts * DKPT, ch = part * DKPT;
    float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride + (static_cast<size_t>(h) * dv + c) * dkp + ch;
    float S[DKPT];
    {
        const float4 a = *reinterpret_cast<const float4*>(srow), d = *reinterpret_cast<const float4*>(srow + 4);
        S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = d.x; S[5] = d.y; S[6] = d.z; S[7] = d.w;
    }
    const float w = decay[h];
    const int q_off = h * dk, k_off = H * dk + h * dk, v_off = 2 * H * dk + h * dv + c;
    const bool whole = dk % DKPT == 0 && ch + DKPT <= dk && act_stride % 4 == 0;
    const bool idle = ch >= dk;                   // a lane that holds padding only
    const int t0 = q_start[b];
    DecayOperands cur, nxt;
    if (!idle) decay_load(cur, act + static_cast<size_t>(t0) * act_stride, q_off, k_off, v_off, ch, dk, whole);
    for (int r = 0; r < n; ++r) {
        if (!idle && r + 1 < n) decay_load(nxt, act + static_cast<size_t>(t0 + r + 1) * act_stride, q_off, k_off, v_off, ch, dk, whole);
        float sum = 0.f;
        if (!idle) {
#pragma unroll
            for (int i = 0; i < DKPT; ++i) {
                S[i] = w * S[i] + cur.k[i] * cur.v;
                sum += S[i] * cur.q[i];
            }
        }
        sum = parts_sum(sum, parts);
        if (part == 0) out[static_cast<size_t>(t0 + r) * (H * dv) + h * dv + c] = sum;
        cur = nxt;
    }
    if (!idle) {
        *reinterpret_cast<float4*>(srow) = make_float4(S[0], S[1], S[2], S[3]);
        *reinterpret_cast<float4*>(srow + 4) = make_float4(S[4], S[5], S[6], S[7]);
    }
}

NI_EXPORT int ni_decay_attention_parts(int dk) {
    int parts = 1;
    while (parts * DKPT < dk) parts *= 2;
    return parts <= WAVE ? parts : 0;
}

NI_EXPORT int ni_decay_attention(const void* act, int act_stride, const void* decay, void* state, size_t state_stride,
                                 const void* q_start, const void* q_len, const void* state_slot, void* out, int T, int B,
                                 int H, int dk, int dv, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    const int parts = ni_decay_attention_parts(dk);
    if (!parts || act_stride < 2 * H * dk + H * dv || state_stride < static_cast<size_t>(H) * dv * parts * DKPT) return -1;
    if (reinterpret_cast<uintptr_t>(state) % 16 || state_stride % 4 || reinterpret_cast<uintptr_t>(act) % 16) return -1;
    const int cols = 4 * (WAVE / parts);
    dim3 grid((dv + cols - 1) / cols, H, B);
    decay_attention_kernel<<<grid, 256, 0, stream>>>((const float*)act, act_stride, (const float*)decay, (float*)state, state_stride,
                                                     (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot,
                                                     (float*)out, H, dk, dv, parts);
    return NI_LAUNCH_RESULT();
}

// y[t, :] = o[t, :] / sqrt(mean(o[t, :]^2) + eps) * w * sigmoid(gate[t, :]) * out_scale, in the type T.
// One workgroup a token; gate rows have a stride of their own (they are columns of a wider projection).
template <typename T>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ gate, int gate_stride, const float* __restrict__ w,
                     T* __restrict__ y, int n, float eps, float out_scale) {
    __shared__ float scratch[8];
    const int t = blockIdx.x;
    const float* row = o + static_cast<size_t>(t) * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss += row[i] * row[i];
    const float r = out_scale / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
    const float* g = gate + static_cast<size_t>(t) * gate_stride;
    for (int i = threadIdx.x; i < n; i += blockDim.x) st(y + static_cast<size_t>(t) * n + i, row[i] * r * w[i] * sigmoid_f(g[i]));
}

NI_EXPORT int ni_gated_rmsnorm(const void* o, const void* gate, int gate_stride, const void* w, void* y, int T, int n, float eps,
                               float out_scale, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (gate_stride < n) return -1;
    if (dtype == 0)
        gated_rmsnorm_kernel<float><<<T, 256, 0, stream>>>((const float*)o, (const float*)gate, gate_stride, (const float*)w, (float*)y, n, eps, out_scale);
    else
        gated_rmsnorm_kernel<bf16_t><<<T, 256, 0, stream>>>((const float*)o, (const float*)gate, gate_stride, (const float*)w, (bf16_t*)y, n, eps, out_scale);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- causal convolution per channel, then silu
//   u[t, c] = silu(bias[c] + sum_j w[c, j] * x[t - (taps - 1 - j), c])      the last tap is the token's own input
// x is the first `inner` columns of xz float32 [T, xz_stride].  Inputs before a portion's first row come from
// `tail` (per slot [(taps - 1)][inner], the oldest first; zero for a new sequence), which conv_tail_kernel moves on
// afterwards, in a launch of its own.  u goes out as float32 (for the recurrence) and, if asked for, in the compute
// type (for the product that follows).
template <typename T>
__global__ void conv_silu_kernel(const float* __restrict__ xz, int xz_stride, const float* __restrict__ w, const float* __restrict__ bias,
                                 const float* __restrict__ state, size_t state_stride, size_t tail_off,
                                 const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
                                 const int32_t* __restrict__ state_slot, float* __restrict__ u32, T* __restrict__ uc,
                                 int inner, int taps, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / inner), c = static_cast<int>(i % inner);
    const int b = seq_of_token[t];
    const int r = t - q_start[b];                 // place of the token in its portion
    const float* tail = state + static_cast<size_t>(state_slot[b]) * state_stride + tail_off;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;            // how many tokens before this one
        const float x = r - back >= 0 ? xz[static_cast<size_t>(t - back) * xz_stride + c]
                                      : tail[static_cast<size_t>(taps - 1 + r - back) * inner + c];
        acc += w[static_cast<size_t>(c) * taps + j] * x;
    }
    const float v = silu_f(acc);
    u32[i] = v;
    if (uc) st(uc + i, v);
}

// the last taps - 1 inputs of every sequence of the step, oldest first; a thread moves one channel's column
__global__ void conv_tail_kernel(const float* __restrict__ xz, int xz_stride, float* __restrict__ state, size_t state_stride,
                                 size_t tail_off, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                 const int32_t* __restrict__ state_slot, int inner, int taps, int B) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= inner || b >= B) return;
    const int n = q_len[b], keep = taps - 1;
    if (n <= 0) return;
    float* tail = state + static_cast<size_t>(state_slot[b]) * state_stride + tail_off;
    for (int j = 0; j < keep; ++j) {              // ascending: what is read lies at or above what has been written
        const int idx = n - keep + j;             // place in the portion of the input that ends up at j
        tail[static_cast<size_t>(j) * inner + c] = idx >= 0 ? xz[static_cast<size_t>(q_start[b] + idx) * xz_stride + c]
                                                            : tail[static_cast<size_t>(keep + idx) * inner + c];
    }
}

NI_EXPORT int ni_conv_silu(const void* xz, int xz_stride, const void* w, const void* bias, void* state, size_t state_stride,
                           size_t tail_off, const void* seq_of_token, const void* q_start, const void* q_len, const void* state_slot,
                           void* u32, void* uc, int T, int B, int inner, int taps, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * inner;
    if (total == 0 || B <= 0) return 0;
    if (taps < 1 || xz_stride < inner || state_stride < tail_off + static_cast<size_t>(taps - 1) * inner) return -1;
    if (dtype == 0)
        conv_silu_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)xz, xz_stride, (const float*)w, (const float*)bias,
            (const float*)state, state_stride, tail_off, (const int32_t*)seq_of_token, (const int32_t*)q_start, (const int32_t*)state_slot,
            (float*)u32, (float*)uc, inner, taps, total);
    else
        conv_silu_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)xz, xz_stride, (const float*)w, (const float*)bias,
            (const float*)state, state_stride, tail_off, (const int32_t*)seq_of_token, (const int32_t*)q_start, (const int32_t*)state_slot,
            (float*)u32, (bf16_t*)uc, inner, taps, total);
    if (taps > 1) {
        dim3 grid(blocks_of(inner, 256), B);
        conv_tail_kernel<<<grid, 256, 0, stream>>>((const float*)xz, xz_stride, (float*)state, state_stride, tail_off,
                                                   (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot, inner, taps, B);
    }
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the selective scan
//   dt = softplus(dt_pre[t, c] + dt_bias[c])
//   S[c, n] <- exp(dt A[c, n]) S[c, n] + dt u[t, c] B[t, n];   y[t, c] = (sum_n S[c, n] C[t, n] + D[c] u[t, c]) * silu(z[t, c])
// A float32 [inner][np] (negative; the padding zero), bc float32 [T, bc_stride] with B at column 0 and C at column N,
// z a column block of a wider projection (stride z_stride).  The state of a slot is [inner][np], np = parts * 4 >= N.
// A channel is held by `parts` neighbouring lanes with four of its numbers each; y in the type T.
#define SNPT 4

struct ScanOperands {
    float dt_pre, u, z, B[SNPT], C[SNPT];
};

__device__ __forceinline__ void scan_load(ScanOperands& o, const float* __restrict__ dt_pre, const float* __restrict__ u,
                                          const float* __restrict__ z, int z_stride, const float* __restrict__ bc, int bc_stride,
                                          size_t t, int c, int inner, int n0, int N, bool whole) {
    o.dt_pre = dt_pre[t * inner + c];
    o.u = u[t * inner + c];
    o.z = z[t * z_stride + c];
    const float* row = bc + t * bc_stride;
    if (whole) {
        const float4 a = *reinterpret_cast<const float4*>(row + n0), b = *reinterpret_cast<const float4*>(row + N + n0);
        o.B[0] = a.x; o.B[1] = a.y; o.B[2] = a.z; o.B[3] = a.w;
        o.C[0] = b.x; o.C[1] = b.y; o.C[2] = b.z; o.C[3] = b.w;
    } else {
#pragma unroll
        for (int i = 0; i < SNPT; ++i) {
            const bool in = n0 + i < N;
            o.B[i] = in ? row[n0 + i] : 0.f;
            o.C[i] = in ? row[N + n0 + i] : 0.f;
        }
    }
}

template <typename T>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const float* __restrict__ dt_pre, const float* __restrict__ dt_bias, const float* __restrict__ u,
                      const float* __restrict__ z, int z_stride, const float* __restrict__ bc, int bc_stride,
                      const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state, size_t state_stride,
                      const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot,
                      T* __restrict__ y, int inner, int N, int parts) {
    const int b = blockIdx.y;
    const int part = threadIdx.x % parts;
    const int c = (blockIdx.x * blockDim.x + threadIdx.x) / parts;
    const int n = q_len[b];
    if (c >= inner || n <= 0) return;            // whole groups of `parts` lanes leave together
    const int np = parts * SNPT, n0 = part * SNPT;
    float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride + static_cast<size_t>(c) * np + n0;
    const float4 s4 = *reinterpret_cast<const float4*>(srow);
    float S[SNPT] = {s4.x, s4.y, s4.z, s4.w};
    const float4 a4 = *reinterpret_cast<const float4*>(A + static_cast<size_t>(c) * np + n0);
    const float Ac[SNPT] = {a4.x, a4.y, a4.z, a4.w};
    const float bias = dt_bias[c], Dc = D[c];
    const bool whole = N % SNPT == 0 && n0 + SNPT <= N && bc_stride % 4 == 0;
    const size_t t0 = static_cast<size_t>(q_start[b]);
    ScanOperands cur, nxt;
    scan_load(cur, dt_pre, u, z, z_stride, bc, bc_stride, t0, c, inner, n0, N, whole);
    for (int r = 0; r < n; ++r) {
        if (r + 1 < n) scan_load(nxt, dt_pre, u, z, z_stride, bc, bc_stride, t0 + r + 1, c, inner, n0, N, whole);
        const float dt = softplus_f(cur.dt_pre + bias);
        const float du = dt * cur.u;
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < SNPT; ++i) {
            S[i] = expf(dt * Ac[i]) * S[i] + du * cur.B[i];
            sum += S[i] * cur.C[i];
        }
        sum = parts_sum(sum, parts);
        if (part == 0) st(y + (t0 + r) * inner + c, (sum + Dc * cur.u) * silu_f(cur.z));
        cur = nxt;
    }
    *reinterpret_cast<float4*>(srow) = make_float4(S[0], S[1], S[2], S[3]);
}

NI_EXPORT int ni_selective_scan_parts(int N) {
    int parts = 1;
    while (parts * SNPT < N) parts *= 2;
    return parts <= WAVE ? parts : 0;
}

NI_EXPORT int ni_selective_scan(const void* dt_pre, const void* dt_bias, const void* u, const void* z, int z_stride, const void* bc,
                                int bc_stride, const void* A, const void* D, void* state, size_t state_stride, const void* q_start,
                                const void* q_len, const void* state_slot, void* y, int T, int B, int inner, int N, int dtype,
                                hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    const int parts = ni_selective_scan_parts(N);
    if (!parts || z_stride < inner || bc_stride < 2 * N || state_stride < static_cast<size_t>(inner) * parts * SNPT) return -1;
    if (reinterpret_cast<uintptr_t>(state) % 16 || state_stride % 4 || reinterpret_cast<uintptr_t>(A) % 16 ||
        reinterpret_cast<uintptr_t>(bc) % 16) return -1;
    dim3 grid(blocks_of(static_cast<size_t>(inner) * parts, 256), B);
    if (dtype == 0)
        selective_scan_kernel<float><<<grid, 256, 0, stream>>>((const float*)dt_pre, (const float*)dt_bias, (const float*)u, (const float*)z,
            z_stride, (const float*)bc, bc_stride, (const float*)A, (const float*)D, (float*)state, state_stride, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, (float*)y, inner, N, parts);
    else
        selective_scan_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)dt_pre, (const float*)dt_bias, (const float*)u, (const float*)z,
            z_stride, (const float*)bc, bc_stride, (const float*)A, (const float*)D, (float*)state, state_stride, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, (bf16_t*)y, inner, N, parts);
    return NI_LAUNCH_RESULT();
}
