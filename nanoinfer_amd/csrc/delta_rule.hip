// The gated delta rule with one decay per key channel, for gfx950.
//
// Per head, with S [key channel, value channel] float32 carried from token to token:
//     S <- diag(g_t) S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
// Six kernels:
//   delta_prepare      per token, in parallel: the short causal convolutions of q, k, v with silu, the unit
//                      norms of q and k, beta = sigmoid, g = exp(-exp(A) softplus(z + dt)), the output gate
//   conv_state_update  per sequence: the last taps - 1 inputs of the convolutions, kept for the next step
//   delta_rule         per (sequence, head, group of value channels): the recurrence over the step's tokens
//   headnorm_gate      o / rms(o) * w * gate per head, rounded to the compute type for the output product
//   delta_chunk_prepare, delta_chunk_scan   the same recurrence for portions of prompts, sixteen tokens at a
//                      time on the matrix cores (described above them)
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

// Sum over the PARTS neighbouring lanes that hold one column (PARTS a power of two up to 16, aligned: they lie in
// one row of sixteen lanes), every lane getting the total, by data-parallel moves inside the row: pairs, quads, the
// mirrored half, the mirrored row.  No trip through the LDS crossbar stands in the recurrence's chain.
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
template <int N> __device__ __forceinline__ float parts_sum(float v) {
    if constexpr (N >= 2) v += dpp_move<0xB1>(v);       // quad_perm [1, 0, 3, 2]
    if constexpr (N >= 4) v += dpp_move<0x4E>(v);       // quad_perm [2, 3, 0, 1]
    if constexpr (N >= 8) v += dpp_move<0x141>(v);      // row_half_mirror: lane i <-> 7 - i of its eight
    if constexpr (N >= 16) v += dpp_move<0x140>(v);     // row_mirror: lane i <-> 15 - i of its sixteen
    return v;
}

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z * sigmoid_f(z); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// proj float32 [T, proj_cols]: q [G*dk] | k [G*dk] | v [H*dv] | b [H] as projected.
// low float32 [T, H*dk + H*dv]: the decay's pre-activation, then the output gate's.
// conv float32 [C, taps] with C = 2*G*dk + H*dv (the filters of q, k, v stacked).
// state float32 [slots, state_stride]; the convolutions' inputs lie at conv_off as [taps - 1, C].
// prep float32 [T, prep_cols]: q | k | v | beta [H] | g [H*dk] | gate [H*dv].
// One workgroup a (token, unit): units 0 .. 2G-1 are the heads of q and of k (convolution, silu, unit norm),
// units 2G .. 2G+H-1 the heads of v with that head's beta, decay and gate.
__device__ __forceinline__ float conv_at(const float* __restrict__ proj, const float* __restrict__ hist,
                                         const float* __restrict__ conv, int t, int i, int c, int C, int taps, int proj_cols) {
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;
        const float x = (i - back >= 0) ? proj[static_cast<size_t>(t - back) * proj_cols + c]
                                        : hist[static_cast<size_t>(taps - 1 + i - back) * C + c];
        acc += conv[static_cast<size_t>(c) * taps + j] * x;
    }
    return acc;
}

__global__ void delta_prepare_kernel(const float* __restrict__ proj, const float* __restrict__ low,
                                     const float* __restrict__ conv, const float* __restrict__ a_log,
                                     const float* __restrict__ dt_bias, float* __restrict__ state,
                                     const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
                                     const int32_t* __restrict__ state_slot, float* __restrict__ prep,
                                     int G, int H, int dk, int dv, int taps, int proj_cols, size_t state_stride,
                                     size_t conv_off, int log_decay, int move_on) {
    __shared__ float scratch[16];
    const int t = blockIdx.x, unit = blockIdx.y;
    const int s = seq_of_token[t];
    const int i = t - q_start[s];              // place of the token in its portion
    const int QK = 2 * G * dk, C = QK + H * dv;
    const int prep_cols = C + H + H * dk + H * dv;
    float* hist = state + static_cast<size_t>(state_slot[s]) * state_stride + conv_off;
    float* out = prep + static_cast<size_t>(t) * prep_cols;
    // move_on: every sequence of the step brings one token, so the thread that has read a channel's last inputs is the
    // only one that does, and moves them on itself (no kernel of its own for that)
    auto moved = [&](int c) {
        for (int j = 0; j + 2 < taps; ++j) hist[static_cast<size_t>(j) * C + c] = hist[static_cast<size_t>(j + 1) * C + c];
        hist[static_cast<size_t>(taps - 2) * C + c] = proj[static_cast<size_t>(t) * proj_cols + c];
    };
    if (unit < 2 * G) {
        // a head of q or of k: every thread keeps its channels (dk <= 256 = threads)
        const int c = unit * dk + threadIdx.x;
        float y = 0.f;
        if (threadIdx.x < dk) {
            const float z = conv_at(proj, hist, conv, t, i, c, C, taps, proj_cols);
            y = z * (1.0f / (1.0f + expf(-z)));
            if (move_on && taps > 1) moved(c);
        }
        const float ss = block_sum(y * y, scratch);
        const float inv = (1.0f / sqrtf(ss + 1e-6f)) * (unit < G ? 1.0f / sqrtf(static_cast<float>(dk)) : 1.0f);
        if (threadIdx.x < dk) out[c] = y * inv;
        return;
    }
    const int h = unit - 2 * G;
    const float* prow = proj + static_cast<size_t>(t) * proj_cols;
    const float* lrow = low + static_cast<size_t>(t) * (H * dk + H * dv);
    for (int j = threadIdx.x; j < dv; j += blockDim.x) {
        const int c = QK + h * dv + j;
        const float z = conv_at(proj, hist, conv, t, i, c, C, taps, proj_cols);
        out[c] = z * (1.0f / (1.0f + expf(-z)));
        if (move_on && taps > 1) moved(c);
        out[C + H + H * dk + h * dv + j] = 1.0f / (1.0f + expf(-lrow[H * dk + h * dv + j]));
    }
    const float rate = expf(a_log[h]);
    for (int j = threadIdx.x; j < dk; j += blockDim.x) {
        const float z = lrow[h * dk + j] + dt_bias[h * dk + j];
        const float lg = -rate * (z > 20.f ? z : log1pf(expf(z)));
        out[C + H + h * dk + j] = log_decay ? lg : expf(lg);      // the chunked form sums logarithms
    }
    if (threadIdx.x == 0) out[C + h] = 1.0f / (1.0f + expf(-prow[C + h]));
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

// One workgroup: COLS = 256 / PARTS value channels of one head of one sequence.  The operands of CHUNK tokens at a
// time (q, k and g of the head, the workgroup's channels of v, beta) are brought into LDS by all threads together
// while the chunk before is worked through: the recurrence itself then waits for no load from memory, which at one
// token after the other would cost a round trip each.
__global__ void __launch_bounds__(256)
delta_rule_kernel(const float* __restrict__ prep, float* __restrict__ state, const int32_t* __restrict__ q_start,
                  const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot, float* __restrict__ o,
                  int G, int H, int dv, size_t state_stride) {
    constexpr int DK = KPT * PARTS, COLS = 256 / PARTS;
    constexpr int CHUNK = DK <= 128 ? 16 : 8;
    constexpr int ROW = 3 * DK + COLS + 1;                    // q | k | g | v of the workgroup's channels | beta
    constexpr int LOADS = (CHUNK * ROW + 255) / 256;
    __shared__ float buf[2][CHUNK * ROW];
    const int s = blockIdx.x, h = blockIdx.y;
    const int part = threadIdx.x % PARTS;
    const int col0 = blockIdx.z * COLS;
    const int lcol = threadIdx.x / PARTS, col = col0 + lcol;
    const bool live = col < dv;
    const int g = h / (H / G);
    const int QK = 2 * G * DK, C = QK + H * dv;
    const int prep_cols = C + H + H * DK + H * dv;
    const int n = q_len[s], first = q_start[s];
    const float* rows = prep + static_cast<size_t>(first) * prep_cols;
    float* S_mem = state + static_cast<size_t>(state_slot[s]) * state_stride +
                   (static_cast<size_t>(h) * dv + (live ? col : 0)) * DK + part * KPT;
    float S[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) S[i] = live ? S_mem[i] : 0.f;

    float stage[LOADS];
    auto fetch = [&](int t0) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int e = threadIdx.x + j * 256;
            const int tok = e / ROW, r = e % ROW;
            float v = 0.f;
            if (e < CHUNK * ROW && t0 + tok < n) {
                const float* row = rows + static_cast<size_t>(t0 + tok) * prep_cols;
                if (r < DK) v = row[g * DK + r];
                else if (r < 2 * DK) v = row[G * DK + g * DK + (r - DK)];
                else if (r < 3 * DK) v = row[C + H + h * DK + (r - 2 * DK)];
                else if (r < 3 * DK + COLS) { if (col0 + (r - 3 * DK) < dv) v = row[QK + h * dv + col0 + (r - 3 * DK)]; }
                else v = row[C + h];
            }
            stage[j] = v;
        }
    };
    auto put = [&](float* dst) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int e = threadIdx.x + j * 256;
            if (e < CHUNK * ROW) dst[e] = stage[j];
        }
    };
    fetch(0);
    put(buf[0]);
    __syncthreads();
    int which = 0;
    for (int t0 = 0; t0 < n; t0 += CHUNK) {
        const bool more = t0 + CHUNK < n;
        if (more) fetch(t0 + CHUNK);
        const float* cur = buf[which];
        const int count = min(CHUNK, n - t0);
        // unrolled, so that the reads from LDS and the products that do not wait for the memory (k . q) of the next
        // tokens stand ahead of the chain S -> S^T k -> u -> S that every token has to wait for
#pragma unroll 4
        for (int tt = 0; tt < count; ++tt) {
            const float* r = cur + tt * ROW;
            float a = 0.f, a1 = 0.f, b = 0.f, kq = 0.f, k[KPT];
#pragma unroll
            for (int i = 0; i < KPT; ++i) {
                const float q = r[part * KPT + i];
                k[i] = r[DK + part * KPT + i];
                S[i] *= r[2 * DK + part * KPT + i];
                if (i & 1) a1 += S[i] * k[i]; else a += S[i] * k[i];      // two chains of half the length
                b += S[i] * q;
                kq += k[i] * q;
            }
            a = parts_sum<PARTS>(a + a1);
            b = parts_sum<PARTS>(b);
            kq = parts_sum<PARTS>(kq);
            const float u = r[3 * DK + COLS] * (r[3 * DK + lcol] - a);
#pragma unroll
            for (int i = 0; i < KPT; ++i) S[i] += k[i] * u;
            if (live && part == 0) o[(static_cast<size_t>(first) + t0 + tt) * (H * dv) + h * dv + col] = b + u * kq;
        }
        if (more) put(buf[which ^ 1]);
        __syncthreads();
        which ^= 1;
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < KPT; ++i) S_mem[i] = S[i];
    }
}

// ------------------------------------------------------------------ sixteen tokens at a time
// Within a run of C = 16 tokens that starts from the memory S0, with L_t the sum of the logarithms of the decays
// of the run's tokens up to t (a vector over the key channels):
//     u_t + beta_t sum_{s<t} A_ts u_s = beta_t (v_t - S0^T (e^{L_t} k_t)),   A_ts = sum_c k_t[c] k_s[c] e^{L_t[c] - L_s[c]}
//     o_t = S0^T (e^{L_t} q_t) + sum_{s<=t} P_ts u_s,                        P_ts = sum_c q_t[c] k_s[c] e^{L_t[c] - L_s[c]}
//     S_C = diag(e^{L_C}) S0 + sum_s (e^{L_C - L_s} k_s) u_s^T
// Every exponent is a difference that is at most zero: nothing is divided by a decay, however small it gets.
// A, P, the inverse Tm = (I + diag(beta) tril(A, -1))^-1 diag(beta) and the three scaled copies of k and q do not
// depend on the memory: delta_chunk_prepare makes them for all runs of the step at once.  What is left for the
// chain from run to run is five small matrix products,
//     W = V - Kt S0;  U = Tm W;  O = Qt S0 + P U;  S <- diag(e^{L_C}) S0 + Kb^T U,
// which delta_chunk_scan does with v_mfma_f32_16x16x4_f32 (true 32-bit products and sums), one workgroup a
// (sequence, head, sixteen value channels) with its [DK, 16] piece of S in the accumulators' layout for the whole
// step.  A lane of that layout holds channels 4 (lane / 16) + r, r = 0..3, of each sixteen; as the second operand
// of a product over channels the four registers are used one after the other, and the first operand is read in
// the matching order (channel 4 (lane / 16) + r at step r), so that S never moves between layouts.
// Tokens past a sequence's end count as k = q = v = 0, beta = 0, decay 1: they leave S as it is.
// Runs are stored by slot = q_start / 16 + sequence + run: no two sequences of a step share one.
typedef float floatx4_t __attribute__((ext_vector_type(4)));
constexpr int RUN = 16;

__host__ __device__ constexpr int chunk_floats(int dk) { return 3 * RUN * dk + 2 * RUN * RUN + dk; }

__global__ void __launch_bounds__(256)
delta_chunk_prepare_kernel(const float* __restrict__ prep, float* __restrict__ chunks, const int32_t* __restrict__ q_start,
                           const int32_t* __restrict__ q_len, int G, int H, int dv) {
    constexpr int DK = KPT * PARTS, LD = DK + 1;
    __shared__ float Ls[RUN * LD], ks[RUN * LD], qs[RUN * LD], As[RUN * (RUN + 1)], betas[RUN];
    const int s = blockIdx.x, h = blockIdx.z;
    const int n = q_len[s], first = q_start[s];
    const int t0 = blockIdx.y * RUN;
    if (t0 >= n) return;
    const int g = h / (H / G);
    const int QK = 2 * G * DK, C = QK + H * dv;
    const int prep_cols = C + H + H * DK + H * dv;
    const size_t slot = static_cast<size_t>(first / RUN + s + blockIdx.y);
    float* out = chunks + (slot * H + h) * chunk_floats(DK);
    const float* rows = prep + static_cast<size_t>(first + t0) * prep_cols;
    for (int e = threadIdx.x; e < RUN * DK; e += 256) {
        const int t = e / DK, c = e % DK;
        const bool valid = t0 + t < n;
        const float* row = rows + static_cast<size_t>(t) * prep_cols;
        Ls[t * LD + c] = valid ? row[C + H + h * DK + c] : 0.f;
        ks[t * LD + c] = valid ? row[G * DK + g * DK + c] : 0.f;
        qs[t * LD + c] = valid ? row[g * DK + c] : 0.f;
    }
    if (threadIdx.x < RUN) betas[threadIdx.x] = t0 + threadIdx.x < n ? rows[static_cast<size_t>(threadIdx.x) * prep_cols + C + h] : 0.f;
    __syncthreads();
    if (threadIdx.x < DK) {
        float run = 0.f;
        for (int t = 0; t < RUN; ++t) {
            run += Ls[t * LD + threadIdx.x];
            Ls[t * LD + threadIdx.x] = run;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < RUN * DK; e += 256) {
        const int t = e / DK, c = e % DK;
        const float lt = Ls[t * LD + c], lc = Ls[(RUN - 1) * LD + c];
        const float grow = expf(lt);
        out[e] = grow * ks[t * LD + c];
        out[RUN * DK + e] = grow * qs[t * LD + c];
        out[2 * RUN * DK + e] = expf(lc - lt) * ks[t * LD + c];
        if (t == RUN - 1) out[3 * RUN * DK + 2 * RUN * RUN + c] = grow;
    }
    {
        const int t = threadIdx.x / RUN, j = threadIdx.x % RUN;
        float a = 0.f, p = 0.f;
        if (j <= t) {
            for (int c = 0; c < DK; ++c) {
                const float w = expf(Ls[t * LD + c] - Ls[j * LD + c]) * ks[j * LD + c];
                a += ks[t * LD + c] * w;
                p += qs[t * LD + c] * w;
            }
        }
        As[t * (RUN + 1) + j] = j < t ? a : 0.f;
        out[3 * RUN * DK + RUN * RUN + t * RUN + j] = j <= t ? p : 0.f;
    }
    __syncthreads();
    if (threadIdx.x < RUN) {
        // column j of (I + diag(beta) tril(A, -1))^-1 diag(beta), from the top down
        const int j = threadIdx.x;
        float x[RUN];
#pragma unroll
        for (int t = 0; t < RUN; ++t) {
            float acc = 0.f;
#pragma unroll
            for (int r = 0; r < t; ++r) acc += As[t * (RUN + 1) + r] * x[r];
            x[t] = (t == j ? betas[j] : 0.f) - betas[t] * acc;
        }
#pragma unroll
        for (int t = 0; t < RUN; ++t) out[3 * RUN * DK + t * RUN + j] = x[t];
    }
}

// What a wavefront reads for one run of tokens: all of it is asked for one run ahead.
template <int KTW> struct RunOperands {
    float4 kt[KTW], qt[KTW], dec[KTW];   // rows (lane % 16) of Kt and Qt, channels 16 kt + 4 (lane / 16) + r; e^{L_C} of these
    float kb[KTW][4];                    // Kb of token 4 (lane / 16) + r, channel 16 kt + lane % 16
    float4 tm, p;                        // row (lane % 16) of Tm and of P, columns 4 (lane / 16) + r
    floatx4_t v;                         // v of token 4 (lane / 16) + r, the lane's value channel
};

// The key channels of a (head, sixteen value channels) are dealt to SCAN_WAVES wavefronts, sixteen at a time: each
// keeps its channels' rows of S and makes its share of Kt S0 and Qt S0.  The shares meet in LDS once a run (two
// buffers in turn, so one barrier a run is enough: a wavefront can be one run ahead of another, never two); every
// wavefront then sums them in the same order, so all hold the same W and U, and moves its own rows of S on.
constexpr int scan_waves(int kt) { return kt % 4 == 0 ? 4 : kt % 2 == 0 ? 2 : 1; }

__global__ void __launch_bounds__(64 * scan_waves(KPT * PARTS / RUN > 0 ? KPT * PARTS / RUN : 1))
delta_chunk_scan_kernel(const float* __restrict__ prep, const float* __restrict__ chunks, float* __restrict__ state,
                        const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                        const int32_t* __restrict__ state_slot, float* __restrict__ o, int G, int H, int dv,
                        size_t state_stride) {
    constexpr int DK = KPT * PARTS, KT = DK / RUN > 0 ? DK / RUN : 1, SW = scan_waves(KT), KTW = KT / SW;
    __shared__ float shares[2][SW][2][4][WAVE];
    const int s = blockIdx.x, h = blockIdx.y;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE), lane = threadIdx.x % WAVE;
    const int i = lane & 15, g4 = lane >> 4;
    const int col = blockIdx.z * RUN + i;
    const bool live = col < dv;
    const int n = q_len[s], first = q_start[s];
    if (n <= 0) return;
    const int QK = 2 * G * DK, C = QK + H * dv;
    const int prep_cols = C + H + H * DK + H * dv;
    const int ch0 = wave * KTW * RUN;                  // the wavefront's first key channel
    float* S_mem = state + static_cast<size_t>(state_slot[s]) * state_stride + (static_cast<size_t>(h) * dv + (live ? col : 0)) * DK + ch0 + 4 * g4;
    floatx4_t S[KTW];
#pragma unroll
    for (int kt = 0; kt < KTW; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) S[kt][r] = live ? S_mem[kt * RUN + r] : 0.f;
    const float* base = chunks + (static_cast<size_t>(first / RUN + s) * H + h) * chunk_floats(DK);
    const size_t per_run = static_cast<size_t>(H) * chunk_floats(DK);
    const float* vcol = prep + static_cast<size_t>(first) * prep_cols + QK + h * dv + (live ? col : 0);

    auto fetch = [&](RunOperands<KTW>& x, int run) {
        const float* ch = base + per_run * run;
        const int t0 = run * RUN;
#pragma unroll
        for (int kt = 0; kt < KTW; ++kt) {
            const int c = ch0 + kt * RUN;
            x.kt[kt] = *reinterpret_cast<const float4*>(ch + i * DK + c + 4 * g4);
            x.qt[kt] = *reinterpret_cast<const float4*>(ch + RUN * DK + i * DK + c + 4 * g4);
            x.dec[kt] = *reinterpret_cast<const float4*>(ch + 3 * RUN * DK + 2 * RUN * RUN + c + 4 * g4);
#pragma unroll
            for (int r = 0; r < 4; ++r) x.kb[kt][r] = ch[2 * RUN * DK + (4 * g4 + r) * DK + c + i];
        }
        x.tm = *reinterpret_cast<const float4*>(ch + 3 * RUN * DK + i * RUN + 4 * g4);
        x.p = *reinterpret_cast<const float4*>(ch + 3 * RUN * DK + RUN * RUN + i * RUN + 4 * g4);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tok = t0 + 4 * g4 + r;
            x.v[r] = (live && tok < n) ? vcol[static_cast<size_t>(tok) * prep_cols] : 0.f;
        }
    };
    auto at = [](const float4& f, int r) { return r == 0 ? f.x : r == 1 ? f.y : r == 2 ? f.z : f.w; };

    const int runs = (n + RUN - 1) / RUN;
    RunOperands<KTW> cur, nxt;
    fetch(cur, 0);
    for (int run = 0; run < runs; ++run) {
        if (run + 1 < runs) fetch(nxt, run + 1);
        floatx4_t w = {0.f, 0.f, 0.f, 0.f}, out = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kt = 0; kt < KTW; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                w = __builtin_amdgcn_mfma_f32_16x16x4f32(at(cur.kt[kt], r), S[kt][r], w, 0, 0, 0);
                out = __builtin_amdgcn_mfma_f32_16x16x4f32(at(cur.qt[kt], r), S[kt][r], out, 0, 0, 0);
            }
        float (*mine)[2][4][WAVE] = shares[run & 1];
        if constexpr (SW > 1) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                mine[wave][0][r][lane] = w[r];
                mine[wave][1][r][lane] = out[r];
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float sum = mine[0][0][r][lane];
#pragma unroll
                for (int j = 1; j < SW; ++j) sum += mine[j][0][r][lane];
                w[r] = sum;
            }
        }
        w = cur.v - w;
        floatx4_t u = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; ++r) u = __builtin_amdgcn_mfma_f32_16x16x4f32(at(cur.tm, r), w[r], u, 0, 0, 0);
#pragma unroll
        for (int kt = 0; kt < KTW; ++kt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) S[kt][r] *= at(cur.dec[kt], r);
#pragma unroll
            for (int r = 0; r < 4; ++r) S[kt] = __builtin_amdgcn_mfma_f32_16x16x4f32(cur.kb[kt][r], u[r], S[kt], 0, 0, 0);
        }
        // the read-out: P U on top of the shares of Qt S0; a wavefront stores the tokens 4 (lane / 16) + r with r its own
        floatx4_t pu = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; ++r) pu = __builtin_amdgcn_mfma_f32_16x16x4f32(at(cur.p, r), u[r], pu, 0, 0, 0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (r % SW != wave) continue;
            float val = pu[r];
            if constexpr (SW > 1) {
#pragma unroll
                for (int j = 0; j < SW; ++j) val += mine[j][1][r][lane];
            } else {
                val += out[r];
            }
            const int tok = run * RUN + 4 * g4 + r;
            if (live && tok < n) o[(static_cast<size_t>(first) + tok) * (H * dv) + h * dv + col] = val;
        }
        cur = nxt;
    }
    if (live) {
#pragma unroll
        for (int kt = 0; kt < KTW; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) S_mem[kt * RUN + r] = S[kt][r];
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
                               int proj_cols, size_t state_stride, size_t conv_off, int log_decay, int max_q_len, hipStream_t stream) {
    if (T <= 0) return 0;
    const int move_on = max_q_len == 1;         // a step of single tokens: the prepare kernel moves the convolutions' inputs on
    if (dk != KPT * PARTS) return -1;
    const int C = 2 * G * dk + H * dv;
    if (dk > 256) return -2;
    const int widest = std::max(dk, std::min(dv, 256));
    delta_prepare_kernel<<<dim3(T, 2 * G + H), (widest + 63) / 64 * 64, 0, stream>>>((const float*)proj, (const float*)low, (const float*)conv,
                                                  (const float*)a_log, (const float*)dt_bias, (float*)state,
                                                  (const int32_t*)seq_of_token, (const int32_t*)q_start,
                                                  (const int32_t*)state_slot, (float*)prep, G, H, dk, dv, taps, proj_cols,
                                                  state_stride, conv_off, log_decay, move_on);
    if (taps > 1 && !move_on) {
        dim3 grid(B, std::max(1, std::min(64, (C + 255) / 256)));
        conv_state_update_kernel<<<grid, 256, 0, stream>>>((const float*)proj, (float*)state, (const int32_t*)q_start,
                                                           (const int32_t*)q_len, (const int32_t*)state_slot, C, taps,
                                                           proj_cols, state_stride, conv_off);
    }
    return NI_LAUNCH_RESULT();
}

// floats of scratch that the chunked form needs per run of sixteen tokens and head (0: this key size has no such form);
// a step of T tokens in B sequences has at most T / 16 + B + 1 run slots
NI_EXPORT int ni_delta_run_floats() { return (KPT * PARTS) % RUN ? 0 : chunk_floats(KPT * PARTS); }

// chunks: null for the token-by-token kernel (prep then holds the decays), else scratch for the chunked form
// (prep then holds the decays' logarithms); max_q_len is the longest portion of the step
NI_EXPORT int ni_delta_rule(const void* prep, void* chunks, void* state, const void* q_start, const void* q_len,
                            const void* state_slot, void* o, const void* norm_w, void* y, int T, int B, int max_q_len, int G,
                            int H, int dk, int dv, float eps, size_t state_stride, int dtype, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (dk != KPT * PARTS) return -1;
    if (chunks) {
        if constexpr ((KPT * PARTS) % RUN == 0) {
            if (max_q_len < 1) return -1;
            const int runs = (max_q_len + RUN - 1) / RUN;
            delta_chunk_prepare_kernel<<<dim3(B, runs, H), 256, 0, stream>>>((const float*)prep, (float*)chunks, (const int32_t*)q_start,
                                                                             (const int32_t*)q_len, G, H, dv);
            delta_chunk_scan_kernel<<<dim3(B, H, (dv + RUN - 1) / RUN), 64 * scan_waves(KPT * PARTS / RUN), 0, stream>>>(
                (const float*)prep, (const float*)chunks, (float*)state, (const int32_t*)q_start, (const int32_t*)q_len,
                (const int32_t*)state_slot, (float*)o, G, H, dv, state_stride);
        } else {
            return -3;
        }
    } else {
        constexpr int COLS = 256 / PARTS;
        dim3 grid(B, H, (dv + COLS - 1) / COLS);
        delta_rule_kernel<<<grid, 256, 0, stream>>>((const float*)prep, (float*)state, (const int32_t*)q_start,
                                                    (const int32_t*)q_len, (const int32_t*)state_slot, (float*)o, G, H, dv,
                                                    state_stride);
    }
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
