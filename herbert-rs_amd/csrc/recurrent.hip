// Kernels of mixers that carry a state of fixed size from token to token instead of keys and
// values: a short causal convolution over time per channel (its last inputs are state), and the
// gated delta rule, a matrix of state a head that every token first decays, then corrects towards
// its value along its key, then reads with its query. Everything here is float32.
//
// A step's tokens are packed over its sequences: row t belongs to sequence seq_of[t], whose rows
// are [seq_starts[i], seq_starts[i + 1]) and whose state lies at slot slots[i].
#include "common.h"
#include <math.h>

HB_MODULE_ERROR_SLOT()

#define HB_MAX_TAPS 16

__device__ __forceinline__ float hb_silu(float z) { return z / (1.0f + expf(-z)); }

// ------------------------------------------- convolution + silu (+ unit vectors a head)
// Channels are the first C columns of the projection's rows, in sections:
//   [n_unit sections of unit_dim channels | plain sections of plain_dim channels]
// y[t, c] = silu(sum_j taps[c, j] * in[t - (K - 1) + j, c]), the inputs before the step's first row
// from the slot's state [K - 1, C] (zeros in a fresh slot). A unit section is then divided by
// sqrt(sum of squares + unit_eps); sections below n_scaled are also multiplied by `scale`.
// One wave a (token, section).
__global__ void __launch_bounds__(HB_WAVE)
conv_silu_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ taps,
                 const float* __restrict__ conv_state, const int* __restrict__ seq_of,
                 const int* __restrict__ seq_starts, const int* __restrict__ slots, float* __restrict__ out,
                 int C, int K, int n_unit, int unit_dim, int n_scaled, float scale, float unit_eps,
                 int plain_dim) {
    const int t = blockIdx.x;
    const int sec = blockIdx.y;
    const int lane = threadIdx.x;
    const bool unit = sec < n_unit;
    const int c0 = unit ? sec * unit_dim : n_unit * unit_dim + (sec - n_unit) * plain_dim;
    const int len = unit ? unit_dim : plain_dim;
    const int seq = seq_of[t];
    const int first = seq_starts[seq];
    const int at = t - first;                     // the token's place among the step's tokens of its sequence
    const float* state = conv_state + (size_t)slots[seq] * (K - 1) * C;
    float* row = out + (size_t)t * C;
    float ss = 0.f;
    for (int d = lane; d < len; d += HB_WAVE) {
        const int c = c0 + d;
        float acc = 0.f;
        for (int j = 0; j < K; ++j) {
            const int s = at - (K - 1) + j;
            const float v = s >= 0 ? proj[(size_t)(first + s) * ld + c] : state[(size_t)(K - 1 + s) * C + c];
            acc = fmaf(taps[(size_t)c * K + j], v, acc);
        }
        const float y = hb_silu(acc);
        row[c] = y;
        ss = fmaf(y, y, ss);
    }
    if (!unit) return;
    ss = hb_wave_sum(ss);
    const float inv = (sec < n_scaled ? scale : 1.0f) / sqrtf(ss + unit_eps);
    for (int d = lane; d < len; d += HB_WAVE) row[c0 + d] *= inv;     // (each lane rescales what it wrote)
}

// The state after the step: the last K - 1 inputs of each sequence, from the step's rows where it
// brought that many, else the old state moved up. One thread a (sequence, channel).
__global__ void conv_state_kernel(const float* __restrict__ proj, int ld, float* __restrict__ conv_state,
                                  const int* __restrict__ seq_starts, const int* __restrict__ slots, int C,
                                  int K) {
    const int seq = blockIdx.x;
    const int c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int first = seq_starts[seq], n = seq_starts[seq + 1] - first;
    float* state = conv_state + (size_t)slots[seq] * (K - 1) * C;
    float keep[HB_MAX_TAPS];
    for (int i = 0; i < K - 1; ++i) {
        const int s = n - (K - 1) + i;
        keep[i] = s >= 0 ? proj[(size_t)(first + s) * ld + c] : state[(size_t)(i + n) * C + c];
    }
    for (int i = 0; i < K - 1; ++i) state[(size_t)i * C + c] = keep[i];
}

extern "C" int hb_conv_silu(const float* proj, int ld, const float* taps, float* conv_state, const int* seq_of,
                            const int* seq_starts, const int* slots, float* out, int T, int B, int C, int K,
                            int n_unit, int unit_dim, int n_scaled, float scale, float unit_eps, int n_plain,
                            int plain_dim, hipStream_t stream) {
    HB_REQUIRE(T > 0 && B > 0 && C > 0, "conv: empty input");
    HB_REQUIRE(K >= 1 && K <= HB_MAX_TAPS, "conv: %d taps, the kernel takes 1 to %d", K, HB_MAX_TAPS);
    HB_REQUIRE(n_unit * unit_dim + n_plain * plain_dim == C && ld >= C, "conv: the sections do not add up to %d channels", C);
    HB_REQUIRE(n_unit + n_plain <= 65535 && B <= 65535, "conv: too many sections or sequences for the grid");
    conv_silu_kernel<<<dim3(T, n_unit + n_plain), HB_WAVE, 0, stream>>>(
        proj, ld, taps, conv_state, seq_of, seq_starts, slots, out, C, K, n_unit, unit_dim, n_scaled, scale,
        unit_eps, plain_dim);
    HB_CHECK_LAUNCH("conv_silu");
    if (K > 1) {
        conv_state_kernel<<<dim3(B, (C + 255) / 256), 256, 0, stream>>>(proj, ld, conv_state, seq_starts, slots, C, K);
        HB_CHECK_LAUNCH("conv_state");
    }
    return 0;
}

// ------------------------------------------------------------------ gated delta rule
// State S [D, V] a (slot, head). For every token of the sequence, in order:
//   S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q        (o sees the token's own write)
// with g = exp(-exp(A_log[h]) * softplus(a + dt_bias[h])) and beta = sigmoid(b), a and b columns of
// the projection's row. The columns of S never meet, and the tokens are a chain: the kernel is as
// fast as one token's step is short. A column is held by LPC lanes (each 32 of its D numbers, in
// registers; LPC = 1, 2, 4 or 8 for D up to 256), a wave holds 64 / LPC columns and walks the
// sequence's tokens; the two dot products a token are summed over a column's lanes by LPC - 1
// exchanges. The token ahead is loaded while the present one is worked on, and g and beta of a
// token do not wait for the chain.
// qkv rows: [kv_heads x D queries | kv_heads x D keys | heads x V values]; head h reads the
// query and key of kv head h / (heads / kv_heads).
#define DELTA_PER 32

template <int LPC>
__device__ __forceinline__ float delta_column_sum(float v) {
#pragma unroll
    for (int off = 1; off < LPC; off <<= 1) v += __shfl_xor(v, off, HB_WAVE);
    return v;
}

template <int LPC>
__global__ void __launch_bounds__(HB_WAVE)
gated_delta_kernel(const float* __restrict__ qkv, int C, const float* __restrict__ proj, int ld, int b_off,
                   int a_off, const float* __restrict__ A_log, const float* __restrict__ dt_bias,
                   float* __restrict__ state, const int* __restrict__ seq_starts, const int* __restrict__ slots,
                   float* __restrict__ out, int kv_heads, int heads, int D, int V) {
    constexpr int COLS = HB_WAVE / LPC;
    const int seq = blockIdx.x, h = blockIdx.y;
    const int lane = threadIdx.x;
    const int part = lane % LPC;                       // which 32 of the column's D numbers
    const int col = blockIdx.z * COLS + lane / LPC;
    const bool live = col < V;
    const int d0 = part * DELTA_PER;
    const int kvh = h / (heads / kv_heads);
    const int first = seq_starts[seq], last = seq_starts[seq + 1];
    float* S_mem = state + ((size_t)slots[seq] * heads + h) * D * V + col;
    float S[DELTA_PER];
    // (numbers beyond D are zeros and stay zeros: their k and q are loaded as zeros)
#pragma unroll
    for (int i = 0; i < DELTA_PER; ++i) S[i] = (live && d0 + i < D) ? S_mem[(size_t)(d0 + i) * V] : 0.f;
    const float rate = -expf(A_log[h]);
    const float bias = dt_bias[h];
    const int q_at = kvh * D + d0, k_at = (kv_heads + kvh) * D + d0, v_at = 2 * kv_heads * D + h * V;
    const bool whole = d0 + DELTA_PER <= D && (D % 4) == 0 && (C % 4) == 0;      // 16-byte loads of this lane's 32

    float kn[DELTA_PER], qn[DELTA_PER], vn = 0.f, an = 0.f, bn = 0.f;
    auto load = [&](int t) {
        const float* row = qkv + (size_t)t * C;
        if (whole) {
#pragma unroll
            for (int i = 0; i < DELTA_PER; i += 4) {
                const float4 kk = *(const float4*)(row + k_at + i);
                const float4 qq = *(const float4*)(row + q_at + i);
                kn[i] = kk.x, kn[i + 1] = kk.y, kn[i + 2] = kk.z, kn[i + 3] = kk.w;
                qn[i] = qq.x, qn[i + 1] = qq.y, qn[i + 2] = qq.z, qn[i + 3] = qq.w;
            }
        } else {
#pragma unroll
            for (int i = 0; i < DELTA_PER; ++i) {
                kn[i] = d0 + i < D ? row[k_at + i] : 0.f;
                qn[i] = d0 + i < D ? row[q_at + i] : 0.f;
            }
        }
        vn = live ? row[v_at + col] : 0.f;
        an = proj[(size_t)t * ld + a_off + h];
        bn = proj[(size_t)t * ld + b_off + h];
    };
    if (first < last) load(first);
    for (int t = first; t < last; ++t) {
        float kc[DELTA_PER], qc[DELTA_PER];
#pragma unroll
        for (int i = 0; i < DELTA_PER; ++i) {
            kc[i] = kn[i];
            qc[i] = qn[i];
        }
        const float vc = vn;
        const float z = an + bias;
        const float softplus = z > 20.f ? z : log1pf(expf(z));
        const float g = expf(rate * softplus);
        const float beta = 1.0f / (1.0f + expf(-bn));
        if (t + 1 < last) load(t + 1);
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < DELTA_PER; ++i) {
            S[i] *= g;
            dot = fmaf(S[i], kc[i], dot);
        }
        dot = delta_column_sum<LPC>(dot);
        const float u = beta * (vc - dot);
        float o = 0.f;
#pragma unroll
        for (int i = 0; i < DELTA_PER; ++i) {
            S[i] = fmaf(kc[i], u, S[i]);
            o = fmaf(S[i], qc[i], o);
        }
        o = delta_column_sum<LPC>(o);
        if (live && part == 0) out[(size_t)t * heads * V + h * V + col] = o;
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DELTA_PER; ++i)
            if (d0 + i < D) S_mem[(size_t)(d0 + i) * V] = S[i];
    }
}

extern "C" int hb_gated_delta(const float* qkv, int C, const float* proj, int ld, int b_off, int a_off,
                              const float* A_log, const float* dt_bias, float* state, const int* seq_starts,
                              const int* slots, float* out, int B, int kv_heads, int heads, int D, int V,
                              hipStream_t stream) {
    HB_REQUIRE(B > 0 && heads > 0 && kv_heads > 0 && heads % kv_heads == 0, "delta rule: %d heads on %d key heads", heads, kv_heads);
    HB_REQUIRE(D > 0 && D <= 256, "delta rule: keys of %d, the kernel takes 1 to 256", D);
    HB_REQUIRE(V > 0 && C == 2 * kv_heads * D + heads * V, "delta rule: %d channels do not fit the heads", C);
    HB_REQUIRE(B <= 65535 && heads <= 65535, "delta rule: too many sequences or heads for the grid");
    const int lpc = D <= 32 ? 1 : D <= 64 ? 2 : D <= 128 ? 4 : 8;
    const int cols = HB_WAVE / lpc;
    const dim3 grid(B, heads, (V + cols - 1) / cols);
#define HB_DELTA(L)                                                                                               \
    gated_delta_kernel<L><<<grid, HB_WAVE, 0, stream>>>(qkv, C, proj, ld, b_off, a_off, A_log, dt_bias, state,     \
                                                        seq_starts, slots, out, kv_heads, heads, D, V)
    if (lpc == 1) HB_DELTA(1);
    else if (lpc == 2) HB_DELTA(2);
    else if (lpc == 4) HB_DELTA(4);
    else HB_DELTA(8);
#undef HB_DELTA
    HB_CHECK_LAUNCH("gated_delta");
    return 0;
}

// ------------------------------------- norm a head, weight, gate: what leaves the recurrence
// y[t, h, :] = o / sqrt(mean(o^2) + eps) * w * silu(gate[t, h, :]); w [V] is shared by the heads,
// the gate's pre-activations are columns [g_off + h V, ...) of the projection's row. One wave a (token, head).
template <class TOut>
__global__ void __launch_bounds__(HB_WAVE)
gated_head_norm_kernel(const float* __restrict__ o, const float* __restrict__ proj, int ld, int g_off,
                       const float* __restrict__ w, TOut* __restrict__ y, int heads, int V, float eps) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* in = o + ((size_t)t * heads + h) * V;
    const float* gate = proj + (size_t)t * ld + g_off + (size_t)h * V;
    TOut* out = y + ((size_t)t * heads + h) * V;
    float ss = 0.f;
    for (int d = lane; d < V; d += HB_WAVE) ss = fmaf(in[d], in[d], ss);
    ss = hb_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)V + eps);
    for (int d = lane; d < V; d += HB_WAVE) out[d] = hb_from_float<TOut>(in[d] * inv * w[d] * hb_silu(gate[d]));
}

extern "C" int hb_gated_head_norm(const float* o, const float* proj, int ld, int g_off, const float* w, void* y,
                                  int y_dtype, int T, int heads, int V, float eps, hipStream_t stream) {
    HB_REQUIRE(T > 0 && heads > 0 && V > 0 && heads <= 65535, "gated norm: empty input or too many heads");
    if (y_dtype == HB_F32)
        gated_head_norm_kernel<float><<<dim3(T, heads), HB_WAVE, 0, stream>>>(o, proj, ld, g_off, w, (float*)y, heads, V, eps);
    else if (y_dtype == HB_BF16)
        gated_head_norm_kernel<bf16><<<dim3(T, heads), HB_WAVE, 0, stream>>>(o, proj, ld, g_off, w, (bf16*)y, heads, V, eps);
    else
        HB_REQUIRE(false, "gated norm: unknown output dtype %d", y_dtype);
    HB_CHECK_LAUNCH("gated_head_norm");
    return 0;
}
