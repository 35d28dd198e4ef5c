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

// ------------------------------------------------ the same attention on the matrix cores (bfloat16 rows)
// A wave takes 16 heads of one token (the rows of its matrix products) and a range of the keys, in
// chunks of 32. Scores: S^T = K Q^T, the chunk's rows straight from memory as operands (a lane: one
// key's 8 consecutive numbers), the query (times the scale) in registers as two bfloat16 halves, high
// and low, so that it keeps 16 bits of mantissa (with the high half alone a test with large queries
// lost a digit). The sums are float32, and so are the softmax and its state, which are a lane's own
// (a lane holds scores of one head only). Weighted sums: O^T = V^T P^T
// with the weights again as high and low halves (they are never rounded to 8 bits), and V^T, the
// chunk's first `rank` numbers a key with the keys along a row, written to LDS from the registers
// that hold them as the scores' operands. The 32 keys
// of a product stand in the order in which the scores' lanes hold them (4 g + i of the first block of
// 16, then of the second), so the weights go from the scores' registers into the next product as they
// are. With more than one range a token the unnormalised sums, maxima and denominators go to scratch
// and a second kernel joins them in the ranges' order.
// Sizes: rank and rot multiples of 32; RB >= rank / 16, KSM >= (rank + rot) / 32.
typedef __bf16 la_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 la_bf16x4 __attribute__((ext_vector_type(4)));
typedef float la_f32x4 __attribute__((ext_vector_type(4)));
#define LA_CHUNK 32
#define LA_VT_STRIDE 36          // bfloat16 a row of V^T in LDS: 32 keys and 8 bytes, so rows start at other banks

__device__ __forceinline__ void la_split(float v, __bf16& hi, __bf16& lo) {
    hi = (__bf16)v;
    lo = (__bf16)(v - (float)hi);
}

template <int RB, int KSM>
__global__ void __launch_bounds__(HB_WAVE)
latent_attention_mfma_kernel(const float* __restrict__ q_full, const bf16* __restrict__ pages,
                             bf16* __restrict__ out, float* __restrict__ part_acc, float* __restrict__ part_ml,
                             const float* __restrict__ gate, int gate_ld, const int* __restrict__ positions,
                             const int* __restrict__ seq_of, const int* __restrict__ slots,
                             const int* __restrict__ page_table, int max_pages, int page_size, int H, int rank,
                             int rot, float scale, int splits, int chunks_per_split) {
    __shared__ __attribute__((aligned(16))) __bf16 Vt[RB * 16 * LA_VT_STRIDE];
    const int HB = (H + 15) / 16;
    const int t = blockIdx.x / HB, hb = blockIdx.x % HB, split = blockIdx.y;
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const int h = hb * 16 + n;
    const bool head = h < H;
    const int pos = positions[t];
    const int* pt = page_table + (size_t)slots[seq_of[t]] * max_pages;
    const int kd = rank + rot, KS = kd / 32, rblocks = rank / 16, vsteps = rank / 32;
    __bf16* vt_w = Vt + (8 * g) * LA_VT_STRIDE + n;          // where this lane's numbers of a key go

    la_bf16x8 qh[KSM], ql[KSM];
    {
        const float* qrow = q_full + ((size_t)t * H + (head ? h : H - 1)) * kd + 8 * g;
#pragma unroll
        for (int ks = 0; ks < KSM; ++ks)
            if (ks < KS) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    __bf16 hi, lo;
                    la_split(qrow[32 * ks + e] * scale, hi, lo);
                    qh[ks][e] = hi;
                    ql[ks][e] = lo;
                }
            }
    }
    const int n_chunks = (pos + LA_CHUNK) / LA_CHUNK;            // chunks that hold a key <= pos
    const int c_begin = split * chunks_per_split;
    const int c_end = n_chunks < c_begin + chunks_per_split ? n_chunks : c_begin + chunks_per_split;
    float m = -INFINITY, l = 0.f;
    la_f32x4 acc[RB];
#pragma unroll
    for (int db = 0; db < RB; ++db) acc[db] = la_f32x4{0.f, 0.f, 0.f, 0.f};

    for (int c = c_begin; c < c_end; ++c) {
        const int j0 = c * LA_CHUNK;
        // the chunk's 32 keys lie in one page (pages hold a multiple of 32 positions)
        const bf16* chunk = pages + ((size_t)pt[j0 / page_size] * page_size + j0 % page_size) * kd;
        la_f32x4 s[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
            s[kb] = la_f32x4{0.f, 0.f, 0.f, 0.f};
            const bf16* krow = chunk + (size_t)(kb * 16 + n) * kd + 8 * g;
#pragma unroll
            for (int ks = 0; ks < KSM; ++ks)
                if (ks < KS) {
                    const la_bf16x8 kv = *(const la_bf16x8*)(krow + 32 * ks);
                    s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, qh[ks], s[kb], 0, 0, 0);
                    s[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kv, ql[ks], s[kb], 0, 0, 0);
                    // the same numbers are the key's part of V^T: key 16 kb + n, numbers 32 ks + 8 g + e
                    if (ks < vsteps) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) vt_w[(32 * ks + e) * LA_VT_STRIDE + 16 * kb] = kv[e];
                    }
                }
            // (the second block's loads stay behind the first block's products: all of a chunk's rows in
            //  flight at once would not fit the registers beside the sums)
            __builtin_amdgcn_sched_barrier(0);
        }
        // s[kb][i]: key j0 + 16 kb + 4 g + i against head n
        float cmax = -INFINITY;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (j0 + 16 * kb + 4 * g + i > pos) s[kb][i] = -INFINITY;
                cmax = fmaxf(cmax, s[kb][i]);
            }
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, HB_WAVE));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, HB_WAVE));
        const float m_new = fmaxf(m, cmax);                     // finite: the chunk holds a key <= pos
        const float corr = expf(m - m_new);
        la_bf16x8 ph, pl;
        float psum = 0.f;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = expf(s[kb][i] - m_new);
                psum += p;
                __bf16 hi, lo;
                la_split(p, hi, lo);
                ph[4 * kb + i] = hi;
                pl[4 * kb + i] = lo;
            }
        l = l * corr + psum;
        m = m_new;
        // (rescaled every time: a branch around this, for chunks that leave the maximum as it is, made the
        //  compiler spill the sums)
#pragma unroll
        for (int db = 0; db < RB; ++db)
#pragma unroll
            for (int i = 0; i < 4; ++i) acc[db][i] *= corr;
        __syncthreads();
#pragma unroll
        for (int db = 0; db < RB; ++db)
            if (db < rblocks) {
                const __bf16* vr = Vt + (db * 16 + n) * LA_VT_STRIDE + 4 * g;
                const uint2 v0 = *(const uint2*)vr, v1 = *(const uint2*)(vr + 16);
                const la_bf16x8 vv = __builtin_bit_cast(la_bf16x8, uint4{v0.x, v0.y, v1.x, v1.y});
                acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, ph, acc[db], 0, 0, 0);
                acc[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vv, pl, acc[db], 0, 0, 0);
                if (db % 8 == 7) __builtin_amdgcn_sched_barrier(0);      // (no more than eight blocks' reads in flight)
            }
        __syncthreads();
    }
    l += __shfl_xor(l, 16, HB_WAVE);
    l += __shfl_xor(l, 32, HB_WAVE);
    if (!head) return;
    // acc[db][i]: number 16 db + 4 g + i of head n's sum
    const size_t row = (size_t)t * H + h;
    if (splits == 1) {
        float w = l > 0.f ? 1.0f / l : 0.f;
        if (gate) w *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_ld + h]));
#pragma unroll
        for (int db = 0; db < RB; ++db)
            if (db < rblocks) {
#pragma unroll
                for (int i = 0; i < 4; ++i) out[row * rank + db * 16 + 4 * g + i] = hb_from_float<bf16>(acc[db][i] * w);
            }
    } else {
        float* pa = part_acc + (row * splits + split) * rank;
#pragma unroll
        for (int db = 0; db < RB; ++db)
            if (db < rblocks) *(la_f32x4*)(pa + db * 16 + 4 * g) = acc[db];
        if (g == 0) {
            part_ml[(row * splits + split) * 2] = m;
            part_ml[(row * splits + split) * 2 + 1] = l;
        }
    }
}

// out[row, :] = sum over the ranges (in order) of their sums, brought to one maximum, over the summed
// denominators, times sigmoid(gate). One block a (token, head).
__global__ void __launch_bounds__(256)
latent_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16* __restrict__ out,
                    const float* __restrict__ gate, int gate_ld, int H, int rank, int splits) {
    __shared__ float share[HB_WAVE + 1];          // the ranges' weights, and the row's factor
    const size_t row = blockIdx.x;
    if (threadIdx.x < HB_WAVE) {
        // lane s holds range s's share (at most 64 ranges)
        const int lane = threadIdx.x;
        const bool has = lane < splits;
        const float ms = has ? part_ml[(row * splits + lane) * 2] : -INFINITY;
        const float ls = has ? part_ml[(row * splits + lane) * 2 + 1] : 0.f;
        const float m = hb_wave_max(ms);
        const float ws = ms > -INFINITY ? expf(ms - m) : 0.f;
        const float l = hb_wave_sum(ls * ws);
        float w = l > 0.f ? 1.0f / l : 0.f;
        if (gate) w *= 1.0f / (1.0f + expf(-gate[(row / H) * gate_ld + row % H]));
        share[lane] = ws;
        if (lane == 0) share[HB_WAVE] = w;
    }
    __syncthreads();
    const float w = share[HB_WAVE];
    const float* pa = part_acc + row * splits * rank;
    for (int d = threadIdx.x; d < rank; d += blockDim.x) {
        float a = 0.f;
        int s2 = 0;
        for (; s2 + 4 <= splits; s2 += 4) {            // (four ranges' loads at a time; summed in the ranges' order)
            const float v0 = pa[(size_t)s2 * rank + d], v1 = pa[(size_t)(s2 + 1) * rank + d];
            const float v2 = pa[(size_t)(s2 + 2) * rank + d], v3 = pa[(size_t)(s2 + 3) * rank + d];
            a = fmaf(v0, share[s2], a);
            a = fmaf(v1, share[s2 + 1], a);
            a = fmaf(v2, share[s2 + 2], a);
            a = fmaf(v3, share[s2 + 3], a);
        }
        for (; s2 < splits; ++s2) a = fmaf(pa[(size_t)s2 * rank + d], share[s2], a);
        out[row * rank + d] = hb_from_float<bf16>(a * w);
    }
}

extern "C" int hb_latent_attention_mfma(const float* q_full, const void* pages, void* out, float* part_acc,
                                        float* part_ml, const float* gate, int gate_ld, const int* positions,
                                        const int* seq_of, const int* slots, const int* page_table, int max_pages,
                                        int page_size, int T, int H, int rank, int rot, float scale, int splits,
                                        int chunks_per_split, hipStream_t stream) {
    HB_REQUIRE(T > 0 && H > 0, "latent attention: empty input");
    HB_REQUIRE(rank > 0 && rank % 32 == 0 && rank <= 512 && rot % 32 == 0 && rank + rot <= 640,
               "latent attention: the matrix-core kernel takes a latent and a rotated part in steps of 32, up to 512 + 128, not %d + %d", rank, rot);
    HB_REQUIRE(page_size % LA_CHUNK == 0, "latent attention: pages of %d positions", page_size);
    HB_REQUIRE(splits >= 1 && splits <= HB_WAVE && chunks_per_split >= 1, "latent attention: %d ranges, the kernels take 1 to 64", splits);
    HB_REQUIRE(splits == 1 || (part_acc && part_ml), "latent attention: ranges need scratch");
    const long long blocks = (long long)T * ((H + 15) / 16);
    HB_REQUIRE(blocks < (1ll << 31), "latent attention: too many tokens for the grid");
    const dim3 grid((unsigned)blocks, splits);
#define LA_LAUNCH(RBV, KSV)                                                                                      \
    latent_attention_mfma_kernel<RBV, KSV><<<grid, HB_WAVE, 0, stream>>>(                                          \
        q_full, (const bf16*)pages, (bf16*)out, part_acc, part_ml, gate, gate_ld, positions, seq_of, slots,      \
        page_table, max_pages, page_size, H, rank, rot, scale, splits, chunks_per_split)
    if (rank <= 128 && rank + rot <= 256) LA_LAUNCH(8, 8);
    else if (rank <= 256 && rank + rot <= 384) LA_LAUNCH(16, 12);
    else LA_LAUNCH(32, 20);
#undef LA_LAUNCH
    HB_CHECK_LAUNCH("latent_attention_mfma");
    if (splits > 1) {
        latent_merge_kernel<<<(unsigned)((long long)T * H), 256, 0, stream>>>(part_acc, part_ml, (bf16*)out, gate, gate_ld, H, rank, splits);
        HB_CHECK_LAUNCH("latent_merge");
    }
    return 0;
}
