// Attention whose keys and values are made from one small latent vector per token (R elements, RMS-normed) and one
// rotated key part (dr elements) that all heads share.  The cache holds exactly these R + dr numbers per token,
// in the key pool's layout with one "head": [page, 1, 64, R + dr]; there is no value pool.
//
// The products with the matrices that expand a latent into a head's keys and values are moved to the query side:
//   score(q, j) = (q_plain . (U_k c_j) + q_rot . r_j) * scale = ([U_k^T q_plain | q_rot] . [c_j | r_j]) * scale
//   out         = U_v (sum_j p_j c_j)
// so the attention itself runs over the cache rows as they lie: every head is a query of R + dr elements against
// one shared key row, and the values are the first R elements of the same row.  Queries and the latent results
// stay in 32-bit between the three launches (latent_prep, head_project, attn_latent).
#include "common.h"
#include "pta_kernels.h"

// One workgroup per token.  q_rows[t] = H * (dn + dr) query elements (row stride q_ld), down_rows[t] = R + dr (row stride ld).
//  - latent c = down[:R] / sqrt(mean(down[:R]^2) + eps) * w_norm -> cache row [0, R)
//  - shared key part down[R:], its first rot->rotary_dim elements rotated by the token's position -> cache row [R, R + dr)
//  - each head's rotated query part, rotated likewise -> q_full[t, h, R:]  (32-bit)
template <typename T>
__global__ void latent_prep_kernel(float* __restrict__ q_full, T* __restrict__ k_pool, const T* __restrict__ q_rows,
                                   long q_ld, const T* __restrict__ down_rows, long ld, const float* __restrict__ w_norm, float eps,
                                   const float* __restrict__ inv_freq, int inv_freq_ld, float cs_scale, int rot_n,
                                   int pairing, const int* __restrict__ token_pos, const int* __restrict__ token_seq,
                                   const int* __restrict__ block_table, int bt_stride, int H, int dn, int dr, int R,
                                   int write_cache) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const int pos = token_pos[m], seq = token_seq[m];
    const T* row = q_rows + (long)m * q_ld;
    const T* down = down_rows + (long)m * ld;
    const float* freq = inv_freq ? inv_freq + (inv_freq_ld ? (long)seq * inv_freq_ld : 0) : nullptr;
    const int D = R + dr;
    // the element that element i of a rotated part is paired with, and the sign of the sine term
    auto rotated = [&](const T* v, int i) -> float {
        const float a = Io<T>::ld(v + i);
        if (!freq || i >= rot_n) return a;
        int pair, fi;
        float sign;
        if (pairing == PTA_PAIR_INTERLEAVED) { pair = i ^ 1; fi = i >> 1; sign = (i & 1) ? 1.f : -1.f; }
        else { const int half = rot_n >> 1; pair = i < half ? i + half : i - half; fi = i < half ? i : i - half; sign = i < half ? -1.f : 1.f; }
        const float ang = (float)pos * freq[fi];
        return a * (cosf(ang) * cs_scale) + sign * Io<T>::ld(v + pair) * (sinf(ang) * cs_scale);
    };
    if (write_cache) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < R; i += blockDim.x) { const float v = Io<T>::ld(down + i); ss += v * v; }
        ss = block_sum(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)R + eps);
        const long page = block_table[(long)seq * bt_stride + pos / PTA_PAGE];
        T* dst = k_pool + (page * PTA_PAGE + pos % PTA_PAGE) * (long)D;
        for (int i = threadIdx.x; i < R; i += blockDim.x) Io<T>::st(dst + i, Io<T>::ld(down + i) * inv * w_norm[i]);
        for (int i = threadIdx.x; i < dr; i += blockDim.x) Io<T>::st(dst + R + i, rotated(down + R, i));
    }
    for (int i = threadIdx.x; i < H * dr; i += blockDim.x) {
        const int h = i / dr, e = i - h * dr;
        q_full[((long)m * H + h) * D + R + e] = rotated(row + (long)h * (dn + dr) + dn, e);
    }
}

// q_rows [M, H * (dn + dr)] rows q_ld apart; down_rows [M, R + dr] rows ld apart (the two may be blocks of columns of
// one product, or come from two)
extern "C" int pta_latent_prep(float* q_full, void* k_pool, const void* q_rows, long q_ld, const void* proj, long ld,
                               const float* w_norm, float eps,
                               const PtaRotation* rot, const int* token_pos, const int* token_seq,
                               const int* block_table, int bt_stride, int M, int H, int dn, int dr, int R,
                               int write_cache, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && dn > 0 && dr >= 0 && R > 0, "latent_prep: sizes must be positive");
    PTA_REQUIRE(q_full && k_pool && q_rows && proj && w_norm && token_pos && token_seq && block_table, "latent_prep: null pointer");
    PTA_REQUIRE(q_ld >= (long)H * (dn + dr) && ld >= (long)R + dr, "latent_prep: rows lie closer together than they are long");
    const float* inv_freq = rot ? rot->inv_freq : nullptr;
    int rot_n = 0, pairing = PTA_PAIR_HALF, freq_ld = 0;
    float cs = 1.f;
    if (inv_freq) {
        rot_n = rot->rotary_dim, pairing = rot->pairing, freq_ld = rot->inv_freq_ld, cs = rot->cs_scale;
        PTA_REQUIRE(rot_n >= 2 && rot_n % 2 == 0 && rot_n <= dr,
                    "latent_prep: %d rotated elements must be even and at most the rotated part's %d", rot_n, dr);
        PTA_REQUIRE(pairing == PTA_PAIR_HALF || pairing == PTA_PAIR_INTERLEAVED, "latent_prep: unknown pairing %d", pairing);
    }
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(latent_prep_kernel<float>, dim3(M), dim3(256), 0, s, q_full, (float*)k_pool, (const float*)q_rows,
                           q_ld, (const float*)proj, ld, w_norm, eps, inv_freq, freq_ld, cs, rot_n, pairing, token_pos, token_seq, block_table,
                           bt_stride, H, dn, dr, R, write_cache);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(latent_prep_kernel<bf16_t>, dim3(M), dim3(256), 0, s, q_full, (bf16_t*)k_pool,
                           (const bf16_t*)q_rows, q_ld, (const bf16_t*)proj, ld, w_norm, eps, inv_freq, freq_ld, cs, rot_n, pairing, token_pos,
                           token_seq, block_table, bt_stride, H, dn, dr, R, write_cache);
    else
        return pta_fail("latent_prep: unknown dtype %d", dtype);
    return pta_check_launch("latent_prep");
}

// A small product per head: out[t, h, o] = sum_k in[t, h, k] * W[h][k, o], with head h's matrix at w + h * K * O,
// K-major (its rows are inputs), so that neighbouring threads read neighbouring outputs.
// A workgroup of eight waves owns (16 tokens, head, 64 outputs); K is walked in pieces of 512 that lie in LDS, a wave
// takes an eighth of a piece with all its loads of W in flight at once, and the waves add up in LDS in wave order.
// For steps of few tokens; prompts in bfloat16 go to the vendor library's batched product instead.
#define HP_WAVES 8
#define HP_PIECE 512
#define HP_PER (HP_PIECE / HP_WAVES)

template <typename TI, typename TW, typename TO>
__global__ __launch_bounds__(64 * HP_WAVES) void head_project_kernel(TO* __restrict__ out, long out_ld, long out_head,
                                                                     const TI* __restrict__ in, long in_ld, long in_head,
                                                                     const TW* __restrict__ w, int M, int K, int O) {
    __shared__ float in_s[16][HP_PIECE + 1];
    __shared__ float part[HP_WAVES - 1][16][64];
    const int h = blockIdx.y, m0 = blockIdx.z * 16, lane = threadIdx.x & 63, o = blockIdx.x * 64 + lane, kq = threadIdx.x >> 6;
    float acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.f;
    for (int k0 = 0; k0 < K; k0 += HP_PIECE) {
        const int kc = min(HP_PIECE, K - k0);
        __syncthreads();
        for (int i = threadIdx.x; i < 16 * kc; i += 64 * HP_WAVES) {
            const int t = i / kc, k = i - t * kc;
            in_s[t][k] = m0 + t < M ? Io<TI>::ld(in + (long)(m0 + t) * in_ld + (long)h * in_head + k0 + k) : 0.f;
        }
        __syncthreads();
        if (o < O) {
            const int ka = kq * HP_PER;
            const TW* wp = w + ((long)h * K + k0 + ka) * O + o;
            float wv[HP_PER];
#pragma unroll
            for (int k = 0; k < HP_PER; ++k) wv[k] = ka + k < kc ? Io<TW>::ld(wp + (long)k * O) : 0.f;
#pragma unroll
            for (int k = 0; k < HP_PER; ++k) {
                if (ka + k < kc) {
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc[i] += in_s[i][ka + k] * wv[k];
                }
            }
        }
    }
    if (kq > 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) part[kq - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (kq == 0 && o < O) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int t = m0 + i;
            float v = acc[i];
#pragma unroll
            for (int q = 0; q < HP_WAVES - 1; ++q) v += part[q][i][lane];
            if (t < M) Io<TO>::st(out + (long)t * out_ld + (long)h * out_head + o, v);
        }
    }
}

// in_wide / out_wide: the activations on that side are 32-bit whatever `dtype` (the type of w) says
extern "C" int pta_head_project(void* out, int out_wide, long out_ld, long out_head, const void* in, int in_wide,
                                long in_ld, long in_head, const void* w, int M, int H, int K, int O, int dtype,
                                void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && K > 0 && O > 0, "head_project: sizes must be positive");
    PTA_REQUIRE(out && in && w, "head_project: null pointer");
    PTA_REQUIRE(H <= 65535 && (M + 15) / 16 <= 65535, "head_project: too many heads or tokens for one launch");
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((O + 63) / 64, H, (M + 15) / 16), block(64 * HP_WAVES);
#define HP_LAUNCH(TI, TW, TO) hipLaunchKernelGGL((head_project_kernel<TI, TW, TO>), grid, block, 0, s, (TO*)out, out_ld, out_head, \
                                                 (const TI*)in, in_ld, in_head, (const TW*)w, M, K, O)
    if (dtype == PTA_F32) HP_LAUNCH(float, float, float);
    else if (dtype != PTA_BF16) return pta_fail("head_project: unknown dtype %d", dtype);
    else if (in_wide && out_wide) HP_LAUNCH(float, bf16_t, float);
    else if (in_wide) HP_LAUNCH(float, bf16_t, bf16_t);
    else if (out_wide) HP_LAUNCH(bf16_t, bf16_t, float);
    else HP_LAUNCH(bf16_t, bf16_t, bf16_t);
#undef HP_LAUNCH
    return pta_check_launch("head_project");
}

// Causal attention of every token over its sequence's cache rows, all arithmetic in 32-bit.  One wave per (token,
// head); keys a page of 64 at a time from position 0 in a running softmax, so what a token computes does not
// depend on how the sequence was cut into steps or on the rest of the batch.  q [M, H, D] and out [M, H, R]
// are 32-bit; a cache row is [R + dr] of the compute type, and its first R elements are the value.
#define LAT_MAX_ACC 8  // R <= 64 * LAT_MAX_ACC

template <typename T>
__global__ void attn_latent_kernel(float* __restrict__ out, const float* __restrict__ q, const T* __restrict__ k_pool,
                                   const int* __restrict__ block_table, int bt_stride, const int* __restrict__ token_seq,
                                   const int* __restrict__ token_pos, int H, int R, int D, float scale) {
    extern __shared__ float q_s[];  // [D], then the page's weights [64]
    float* p_s = q_s + D;
    const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int seq = token_seq[m];
    const int nkeys = token_pos[m] + 1;
    const int* bt = block_table + (long)seq * bt_stride;
    const float* qr = q + ((long)m * H + h) * D;
    for (int i = lane; i < D; i += PTA_WAVE) q_s[i] = qr[i] * scale;
    __syncthreads();
    float m_run = -INFINITY, l_run = 0.f;
    float acc[LAT_MAX_ACC];
#pragma unroll
    for (int r = 0; r < LAT_MAX_ACC; ++r) acc[r] = 0.f;
    for (int c0 = 0; c0 < nkeys; c0 += PTA_PAGE) {
        const long page = bt[c0 / PTA_PAGE];
        const T* kp = k_pool + page * (long)PTA_PAGE * D;
        const bool valid = c0 + lane < nkeys;
        float s = -INFINITY;
        if (valid) {
            const T* kr = kp + (long)lane * D;
            float dot = 0.f;
            for (int i = 0; i < D; ++i) dot += q_s[i] * Io<T>::ld(kr + i);
            s = dot;
        }
        const float m_new = fmaxf(m_run, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m_run - m_new);  // 0 on the first page
        l_run = l_run * corr + wave_sum(p);
        __syncthreads();
        p_s[lane] = p;
        __syncthreads();
        const int cnt = min(PTA_PAGE, nkeys - c0);
#pragma unroll
        for (int r = 0; r < LAT_MAX_ACC; ++r) {
            const int dim = lane + r * PTA_WAVE;
            if (dim < R) {
                float a = acc[r] * corr;
                for (int jj = 0; jj < cnt; ++jj) a += p_s[jj] * Io<T>::ld(kp + (long)jj * D + dim);
                acc[r] = a;
            }
        }
        m_run = m_new;
    }
    float* orow = out + ((long)m * H + h) * R;
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int r = 0; r < LAT_MAX_ACC; ++r) {
        const int dim = lane + r * PTA_WAVE;
        if (dim < R) orow[dim] = acc[r] * inv;
    }
}

// Whether the latent attention launches take these sizes (0), or why not (pta_last_error).
extern "C" int pta_attn_latent_sizes_ok(int H, int dn, int dr, int R) {
    PTA_REQUIRE(H > 0 && H <= 65535, "latent attention: %d heads are outside 1..65535", H);
    PTA_REQUIRE(dn > 0 && dr >= 0, "latent attention: head sizes must be positive (plain %d, rotated %d)", dn, dr);
    PTA_REQUIRE(R > 0 && R <= 64 * LAT_MAX_ACC, "latent attention: a latent of %d elements is outside 1..%d", R, 64 * LAT_MAX_ACC);
    return 0;
}

extern "C" int pta_attn_latent(float* out, const float* q, const void* k_pool, const int* block_table, int bt_stride,
                               const int* token_seq, const int* token_pos, int M, int H, int R, int dr, float scale,
                               int dtype, void* stream) {
    PTA_REQUIRE(M > 0, "attn_latent: no tokens");
    if (pta_attn_latent_sizes_ok(H, 1, dr, R)) return 1;
    PTA_REQUIRE(out && q && k_pool && block_table && token_seq && token_pos, "attn_latent: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const int D = R + dr;
    const dim3 grid(M, H), block(PTA_WAVE);
    const size_t lds = (size_t)(D + PTA_PAGE) * sizeof(float);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(attn_latent_kernel<float>, grid, block, lds, s, out, q, (const float*)k_pool, block_table,
                           bt_stride, token_seq, token_pos, H, R, D, scale);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(attn_latent_kernel<bf16_t>, grid, block, lds, s, out, q, (const bf16_t*)k_pool, block_table,
                           bt_stride, token_seq, token_pos, H, R, D, scale);
    else
        return pta_fail("attn_latent: unknown dtype %d", dtype);
    return pta_check_launch("attn_latent");
}
