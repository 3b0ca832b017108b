// Causal attention over the paged cache whose scores pass, before the softmax, through a cap and a mix of the heads:
//
//   s_h(i, j) = q_h(i) . k(j) * scale
//   s_h <- softcap * tanh(s_h / softcap)              (softcap > 0)
//   s_h <- sum over g of talk[h, g] * s_g             (talk given: [heads, heads], 32-bit)
//   weights: softmax over the keys j that i sees (all before it, the last `window`, or its own block of `chunk`)
//   (head_scale given: s_h is multiplied by head_scale[h] before the cap.  weights_kind PTA_WEIGHTS_SIGMOID: a key's
//    weight is sigmoid(s_h + head_bias[h]), not normalised over the keys, in place of the softmax)
//
// The mix needs every head's score of a (query, key) pair in one place: a workgroup owns a token and all of its heads,
// a wave a few heads.  Keys are taken a page (64) at a time from the first page the token sees, a lane a key; the
// capped scores of all heads meet in LDS, every wave mixes its own heads' rows out of them and goes on with a running
// softmax.  All arithmetic is 32-bit, and what a token computes depends on neither the step's cut nor the batch.
// This is the 32-bit path, the path of decode steps and the fallback of prompts.
#include "common.h"
#include "pta_kernels.h"

#define TALK_MAX_WAVES 16

template <typename T, int HPW>
__global__ __launch_bounds__(1024) void attn_talk_kernel(T* __restrict__ out, const T* __restrict__ q,
                                                         const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                                                         const int* __restrict__ block_table, int bt_stride,
                                                         const int* __restrict__ token_seq, const int* __restrict__ token_pos,
                                                         const float* __restrict__ talk, float softcap, int nh, int nkv, int d,
                                                         float scale, int window, int chunk,
                                                         const float* __restrict__ head_scale,
                                                         const float* __restrict__ head_bias, int weights_kind) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float* q_s = sm;                    // [nh][d]
    float* raw_s = q_s + nh * d;        // [nh][64] capped scores of the page
    float* p_s = raw_s + nh * PTA_PAGE; // [nh][64] weights of the page
    float* t_s = p_s + nh * PTA_PAGE;   // [nh][nh]
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int seq = token_seq[m];
    const int nkeys = token_pos[m] + 1;
    const int* bt = block_table + (long)seq * bt_stride;
    const T* qr = q + (long)m * nh * d;
    for (int i = threadIdx.x; i < nh * d; i += blockDim.x) q_s[i] = Io<T>::ld(qr + i);
    if (talk)
        for (int i = threadIdx.x; i < nh * nh; i += blockDim.x) t_s[i] = talk[i];
    __syncthreads();
    int first = window > 0 ? max(0, nkeys - window) : 0;
    if (chunk > 0) first = max(first, (nkeys - 1) / chunk * chunk);
    const int per_kv = nh / nkv;
    const float inv_cap = softcap > 0.f ? 1.0f / softcap : 0.f;
    float m_run[HPW], l_run[HPW], acc[HPW][4];
#pragma unroll
    for (int r = 0; r < HPW; ++r) {
        m_run[r] = -INFINITY;
        l_run[r] = 0.f;
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[r][c] = 0.f;
    }
    for (int c0 = first / PTA_PAGE * PTA_PAGE; c0 < nkeys; c0 += PTA_PAGE) {
        const long page = bt[c0 / PTA_PAGE];
        const int j = c0 + lane;
        const bool valid = j >= first && j < nkeys;
#pragma unroll
        for (int r = 0; r < HPW; ++r) {
            const int h = wave + r * nw;
            if (h < nh) {
                float s = 0.f;
                if (valid) {
                    const T* kr = k_pool + ((page * nkv + h / per_kv) * (long)PTA_PAGE + lane) * d;
                    const float* qh = q_s + h * d;
                    float dot = 0.f;
                    for (int i = 0; i < d; ++i) dot += qh[i] * Io<T>::ld(kr + i);
                    s = dot * scale;
                    if (head_scale) s *= head_scale[h];
                    if (softcap > 0.f) s = softcap * tanhf(s * inv_cap);
                }
                raw_s[h * PTA_PAGE + lane] = s;
            }
        }
        __syncthreads();
        float corr[HPW];
#pragma unroll
        for (int r = 0; r < HPW; ++r) {
            const int h = wave + r * nw;
            corr[r] = 1.f;
            if (h < nh) {
                float s;
                if (talk) {
                    s = 0.f;
                    const float* th = t_s + h * nh;
                    for (int g = 0; g < nh; ++g) s += th[g] * raw_s[g * PTA_PAGE + lane];
                } else {
                    s = raw_s[h * PTA_PAGE + lane];
                }
                if (weights_kind == PTA_WEIGHTS_SIGMOID) {
                    p_s[h * PTA_PAGE + lane] = valid ? 1.0f / (1.0f + expf(-(s + (head_bias ? head_bias[h] : 0.f)))) : 0.f;
                    continue;
                }
                if (!valid) s = -INFINITY;
                const float m_new = fmaxf(m_run[r], wave_max(s));
                const float p = valid ? expf(s - m_new) : 0.f;
                corr[r] = expf(m_run[r] - m_new);  // 0 on the first page
                l_run[r] = l_run[r] * corr[r] + wave_sum(p);
                m_run[r] = m_new;
                p_s[h * PTA_PAGE + lane] = p;
            }
        }
        __syncthreads();
        const int cnt = min(PTA_PAGE, nkeys - c0), j0 = max(0, first - c0);
#pragma unroll
        for (int r = 0; r < HPW; ++r) {
            const int h = wave + r * nw;
            if (h < nh) {
                const T* vp = v_pool + (page * nkv + h / per_kv) * (long)PTA_PAGE * d;
                const float* ph = p_s + h * PTA_PAGE;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int dim = lane + c * PTA_WAVE;
                    if (dim < d) {
                        float a = acc[r][c] * corr[r];
                        for (int jj = j0; jj < cnt; ++jj) a += ph[jj] * Io<T>::ld(vp + (long)dim * PTA_PAGE + jj);
                        acc[r][c] = a;
                    }
                }
            }
        }
        // (the next page's scores overwrite raw_s only after the barrier that follows them; p_s after the one above)
    }
#pragma unroll
    for (int r = 0; r < HPW; ++r) {
        const int h = wave + r * nw;
        if (h < nh) {
            T* orow = out + ((long)m * nh + h) * d;
            const float inv = weights_kind == PTA_WEIGHTS_SIGMOID ? 1.0f : 1.0f / l_run[r];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int dim = lane + c * PTA_WAVE;
                if (dim < d) Io<T>::st(orow + dim, acc[r][c] * inv);
            }
        }
    }
}

// Whether the kernel takes these sizes (0), or why not (pta_last_error).
extern "C" int pta_attn_talk_sizes_ok(int nh, int nkv, int d) {
    PTA_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attn_talk: %d heads are no multiple of %d kv heads", nh, nkv);
    PTA_REQUIRE(d > 0 && d <= 256, "attn_talk: head size %d is outside 1..256", d);
    PTA_REQUIRE(nh <= 4 * TALK_MAX_WAVES, "attn_talk: at most %d heads whose scores are mixed, got %d", 4 * TALK_MAX_WAVES, nh);
    PTA_REQUIRE((size_t)(nh * d + 2 * nh * PTA_PAGE + nh * nh) * 4 <= 64 * 1024,
                "attn_talk: %d heads of %d elements do not fit the kernel's LDS", nh, d);
    return 0;
}

extern "C" int pta_attn_talk(void* out, const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                             int bt_stride, const int* token_seq, const int* token_pos, const float* talk, float softcap, int M,
                             int nh, int nkv, int d, float scale, int window, int chunk, const float* head_scale,
                             const float* head_bias, int weights_kind, int dtype, void* stream) {
    PTA_REQUIRE(weights_kind == PTA_WEIGHTS_SOFTMAX || weights_kind == PTA_WEIGHTS_SIGMOID, "attn_talk: weights of kind %d are not built", weights_kind);
    PTA_REQUIRE(M > 0, "attn_talk: no tokens");
    if (pta_attn_talk_sizes_ok(nh, nkv, d)) return 1;
    PTA_REQUIRE(window >= 0 && chunk >= 0 && softcap >= 0.f, "attn_talk: window, chunk and softcap are 0 (none) or positive");
    PTA_REQUIRE(out && q && k_pool && v_pool && block_table && token_seq && token_pos, "attn_talk: null pointer");
    hipStream_t s = (hipStream_t)stream;
    const int waves = min(nh, TALK_MAX_WAVES), hpw = (nh + waves - 1) / waves;
    const size_t lds = (size_t)(nh * d + 2 * nh * PTA_PAGE + nh * nh) * 4;
#define PTA_TALK(T, R)                                                                                                    \
    hipLaunchKernelGGL((attn_talk_kernel<T, R>), dim3(M), dim3(waves * PTA_WAVE), lds, s, (T*)out, (const T*)q,            \
                       (const T*)k_pool, (const T*)v_pool, block_table, bt_stride, token_seq, token_pos, talk, softcap, nh, \
                       nkv, d, scale, window, chunk, head_scale, head_bias, weights_kind)
#define PTA_TALK_R(T)                       \
    do {                                    \
        if (hpw == 1) PTA_TALK(T, 1);       \
        else if (hpw == 2) PTA_TALK(T, 2);  \
        else PTA_TALK(T, 4);                \
    } while (0)
    if (dtype == PTA_F32) PTA_TALK_R(float);
    else if (dtype == PTA_BF16) PTA_TALK_R(bf16_t);
    else return pta_fail("attn_talk: unknown dtype %d", dtype);
#undef PTA_TALK_R
#undef PTA_TALK
    return pta_check_launch("attn_talk");
}
