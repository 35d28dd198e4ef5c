// Attention whose keys and values of all heads come from one latent vector a token.
// What a token leaves in the cache is one row [c (rank) | r (rot)]: the normed latent and one
// rotated key part that the heads share. Head h's key is [W_uk,h c | r] and its value W_uv,h c; with
// the query's unrotated part taken through W_uk,h^T beforehand (q' = W_uk,h^T q_h, `rank` numbers) the
// score is (q' . c + q_rot . r) * scale, and sum_j p_j c_j (rank numbers) goes through W_uv,h
// afterwards: the kernels here see one shared "key head" of rank + rot numbers whose first `rank`
// are also its value. Scores, softmax and the weighted sums are float32 whatever the storage.
//
// Pages: row of position p of a slot at page_table[slot * max_pages + p / page_size], pages
// [page, page_size, rank + rot].
#include "common.h"
#include <math.h>

HB_MODULE_ERROR_SLOT()

#define HB_MAX_KEY 1152                     // rank + rot
#define HB_MAX_RANK 1024
#define ACC_REGS (HB_MAX_RANK / HB_WAVE)

// the pair (a, b) at angle t: (a cos - b sin, b cos + a sin)
__device__ __forceinline__ void rotate_pair(float a, float b, float angle, float& ra, float& rb) {
    float s, c;
    sincosf(angle, &s, &c);
    ra = a * c - b * s;
    rb = b * c + a * s;
}

// ---------------------------------------- what a token writes: its cache row and its rotated queries
// down (rows down_ld floats apart, as q's are q_ld apart: both may be columns of one projection's rows)
// [T, rank + rot] float32: the first `rank` RMS-normed with norm_w -> the row's c; the last `rot`
// rotated (the first rot_dims of them: entry i with i + rot_dims / 2, angle pos * inv_freq[i]; the rest
// unchanged) -> the row's r. q [T, H, qd + rot] float32: every head's last `rot` rotated the same way
// into q_full[t, h, rank ...] (q_full [T, H, rank + rot] float32; its first `rank` are written by the
// product with W_uk^T). One block a token.
template <class TC>
__global__ void latent_write_kernel(const float* __restrict__ down, int down_ld, const float* __restrict__ norm_w,
                                    const float* __restrict__ q, int q_ld, float* __restrict__ q_full,
                                    bf16* __restrict__ q_plain, const float* __restrict__ inv_freq, const int* __restrict__ positions,
                                    const int* __restrict__ seq_of, const int* __restrict__ slots,
                                    const int* __restrict__ page_table, int max_pages, int page_size,
                                    TC* __restrict__ pages, int H, int qd, int rank, int rot, int rot_dims,
                                    float eps, int write_cache) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int pos = positions[t];
    const int half = rot_dims / 2;
    const float p = (float)pos;
    if (write_cache) {
        const float* in = down + (size_t)t * down_ld;
        float ss = 0.f;
        for (int i = threadIdx.x; i < rank; i += blockDim.x) ss = fmaf(in[i], in[i], ss);
        ss = hb_block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)rank + eps);
        const int slot = slots[seq_of[t]];
        const int page = page_table[(size_t)slot * max_pages + pos / page_size];
        TC* row = pages + ((size_t)page * page_size + pos % page_size) * (rank + rot);
        for (int i = threadIdx.x; i < rank; i += blockDim.x) row[i] = hb_from_float<TC>(in[i] * inv * norm_w[i]);
        for (int i = threadIdx.x; i < rot; i += blockDim.x) {
            float v = in[rank + i];
            if (i < rot_dims) {
                const int j = i < half ? i : i - half;
                float ra, rb;
                rotate_pair(in[rank + j], in[rank + j + half], p * inv_freq[j], ra, rb);
                v = i < half ? ra : rb;
            }
            row[rank + i] = hb_from_float<TC>(v);
        }
    }
    for (int e = threadIdx.x; e < H * rot; e += blockDim.x) {
        const int h = e / rot, i = e % rot;
        const float* in = q + (size_t)t * q_ld + (size_t)h * (qd + rot) + qd;
        float v = in[i];
        if (i < rot_dims) {
            const int j = i < half ? i : i - half;
            float ra, rb;
            rotate_pair(in[j], in[j + half], p * inv_freq[j], ra, rb);
            v = i < half ? ra : rb;
        }
        q_full[((size_t)t * H + h) * (rank + rot) + rank + i] = v;
    }
    // the unrotated parts once more as bfloat16 [T, H, qd], for a matrix-core product with W_uk^T
    if (q_plain)
        for (int e = threadIdx.x; e < H * qd; e += blockDim.x) {
            const int h = e / qd, i = e % qd;
            q_plain[(size_t)t * H * qd + e] = hb_from_float<bf16>(q[(size_t)t * q_ld + (size_t)h * (qd + rot) + i]);
        }
}

extern "C" int hb_latent_write(const float* down, int down_ld, const float* norm_w, const float* q, int q_ld, float* q_full,
                               void* q_plain, const float* inv_freq, const int* positions, const int* seq_of, const int* slots,
                               const int* page_table, int max_pages, int page_size, void* pages, int dtype, int T,
                               int H, int qd, int rank, int rot, int rot_dims, float eps, int write_cache,
                               hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0 && rank > 0 && rot >= 0 && qd >= 0, "latent write: empty input");
    HB_REQUIRE(rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0, "latent write: %d rotated of %d", rot_dims, rot);
    if (dtype == HB_F32)
        latent_write_kernel<float><<<T, 256, 0, stream>>>(down, down_ld, norm_w, q, q_ld, q_full, (bf16*)q_plain, inv_freq, positions, seq_of, slots,
                                                          page_table, max_pages, page_size, (float*)pages, H, qd,
                                                          rank, rot, rot_dims, eps, write_cache);
    else if (dtype == HB_BF16)
        latent_write_kernel<bf16><<<T, 256, 0, stream>>>(down, down_ld, norm_w, q, q_ld, q_full, (bf16*)q_plain, inv_freq, positions, seq_of, slots,
                                                         page_table, max_pages, page_size, (bf16*)pages, H, qd,
                                                         rank, rot, rot_dims, eps, write_cache);
    else
        HB_REQUIRE(false, "latent write: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("latent_write");
    return 0;
}

// ------------------------------------------------ attention over the latent rows, plain
// One wave a (token, head). The keys a query at position p sees are [0, p]; they are walked in
// chunks of 64 that start at multiples of 64 of the absolute position, with an online softmax, so
// the rounding depends on the positions only, not on how the tokens were cut into steps or batches.
// out[t, h, :rank] = sum_j p_j c_j, times sigmoid(gate[t * gate_ld + h]) if a gate is given (the
// head's output is linear in it, so the gate may be applied before W_uv).
template <class TC, class TO>
__global__ void __launch_bounds__(HB_WAVE)
latent_attention_plain_kernel(const float* __restrict__ q_full, const TC* __restrict__ pages,
                              TO* __restrict__ out, const float* __restrict__ gate, int gate_ld,
                              const int* __restrict__ positions, const int* __restrict__ seq_of,
                              const int* __restrict__ slots, const int* __restrict__ page_table, int max_pages,
                              int page_size, int H, int rank, int rot, float scale) {
    __shared__ float qs[HB_MAX_KEY];
    __shared__ float ps[HB_WAVE];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kd = rank + rot;
    const int pos = positions[t];
    const int* pt = page_table + (size_t)slots[seq_of[t]] * max_pages;
    const float* qrow = q_full + ((size_t)t * H + h) * kd;
    for (int d = lane; d < kd; d += HB_WAVE) qs[d] = qrow[d];
    __syncthreads();

    const int hi = pos + 1;
    float m = -INFINITY, l = 0.f;
    float acc[ACC_REGS];
#pragma unroll
    for (int i = 0; i < ACC_REGS; ++i) acc[i] = 0.f;

    for (int c = 0; c < hi; c += HB_WAVE) {
        const int j = c + lane;
        const bool valid = j < hi;
        float s = -INFINITY;
        if (valid) {
            const TC* kr = pages + ((size_t)pt[j / page_size] * page_size + j % page_size) * kd;
            float dot = 0.f;
            for (int d = 0; d < kd; ++d) dot = fmaf(qs[d], hb_to_float(kr[d]), dot);
            s = dot * scale;
        }
        const float m_new = fmaxf(m, hb_wave_max(s));
        const float corr = expf(m - m_new);
        const float p = valid ? expf(s - m_new) : 0.f;
        l = l * corr + hb_wave_sum(p);
        m = m_new;
        __syncthreads();
        ps[lane] = p;
        __syncthreads();
        const int n = hi - c < HB_WAVE ? hi - c : HB_WAVE;
#pragma unroll
        for (int i = 0; i < ACC_REGS; ++i) acc[i] *= corr;
        for (int jj = 0; jj < n; ++jj) {
            const int jv = c + jj;
            const TC* vr = pages + ((size_t)pt[jv / page_size] * page_size + jv % page_size) * kd;
            const float pj = ps[jj];
#pragma unroll
            for (int i = 0; i < ACC_REGS; ++i) {
                const int d = lane + HB_WAVE * i;
                if (d < rank) acc[i] = fmaf(pj, hb_to_float(vr[d]), acc[i]);
            }
        }
    }
    float w = l > 0.f ? 1.0f / l : 0.f;
    if (gate) w *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_ld + h]));
    TO* orow = out + ((size_t)t * H + h) * rank;
#pragma unroll
    for (int i = 0; i < ACC_REGS; ++i) {
        const int d = lane + HB_WAVE * i;
        if (d < rank) orow[d] = hb_from_float<TO>(acc[i] * w);
    }
}

extern "C" int hb_latent_attention_plain(const float* q_full, const void* pages, void* out, int dtype,
                                         const float* gate, int gate_ld, const int* positions, const int* seq_of,
                                         const int* slots, const int* page_table, int max_pages, int page_size,
                                         int T, int H, int rank, int rot, float scale, hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0 && H <= 65535, "latent attention: empty input or too many heads");
    HB_REQUIRE(rank > 0 && rank <= HB_MAX_RANK && rot >= 0 && rank + rot <= HB_MAX_KEY,
               "latent attention: a latent of %d + %d, the kernel takes up to %d + %d", rank, rot, HB_MAX_RANK,
               HB_MAX_KEY - HB_MAX_RANK);
    dim3 grid(T, H);
    if (dtype == HB_F32)
        latent_attention_plain_kernel<float, float><<<grid, HB_WAVE, 0, stream>>>(
            q_full, (const float*)pages, (float*)out, gate, gate_ld, positions, seq_of, slots, page_table, max_pages,
            page_size, H, rank, rot, scale);
    else if (dtype == HB_BF16)
        latent_attention_plain_kernel<bf16, bf16><<<grid, HB_WAVE, 0, stream>>>(
            q_full, (const bf16*)pages, (bf16*)out, gate, gate_ld, positions, seq_of, slots, page_table, max_pages,
            page_size, H, rank, rot, scale);
    else
        HB_REQUIRE(false, "latent attention: unknown dtype %d", dtype);
    HB_CHECK_LAUNCH("latent_attention_plain");
    return 0;
}
