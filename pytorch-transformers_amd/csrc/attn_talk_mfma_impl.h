// Causal attention over the paged cache whose scores are capped and mixed over the heads before the softmax
// (the arithmetic of attn_talk.hip), bfloat16 in, on the matrix cores; prompts and decode steps are the same code.
//
//   s_h(i, j) = q_h(i) . k(j) * scale;  s_h <- cap * tanh(s_h / cap);  s_h <- sum over g of talk[h, g] * s_g
//   (head_scale given: s_h is multiplied by head_scale[h] before the cap.  weights_kind PTA_WEIGHTS_SIGMOID: a key's
//    weight is sigmoid(s_h + head_bias[h]), not normalised over the keys, in place of the softmax)
//
// The mix needs every head's score of a (query, key) pair in one place.  A workgroup owns sixteen consecutive tokens
// of one sequence and all heads (without a mix: the heads of one KV head, or a part of them, heads_wg of them, and
// gridDim.z such workgroups share the tokens); a wave owns CT heads of one KV head.  Keys are walked 32 at a time:
//
//   S_h^T[32 keys x 16 tokens] = K[32 x d] . Q_h^T[d x 16]      per head of the wave, then scale and cap (32-bit)
//   every wave leaves its heads' capped tiles in LDS, in the accumulator's own lane layout; after a barrier it
//   reads all heads' tiles lane by lane and forms the mixed tiles of its own heads: the mix is a product of
//   [heads x heads] with [heads x (token, key) pairs] done on the vector units in 32-bit, nothing changes lanes
//   running softmax per (token, head) in 32-bit; O_h^T[d x 16] += V^T[d x 32] . P_h^T[32 x 16]
//
// The tiles in LDS are double-buffered, so that one barrier per block of keys is enough.  The order of the sum over
// the heads is fixed (0, 1, ...), and the blocks of keys are cut at multiples of 32 of the key's position, so a
// token's result does not depend on how a prompt was cut into steps or on the batch beyond the rounding of the
// running maximum's reference point.
//
// The keys may be cut into ranges, a workgroup per range: with one token per sequence ranges of split_size keys of
// the context; for prompts (split_size 0) every tile's own span of keys in n_splits equal runs of blocks, for launches
// that would otherwise leave compute units idle.  Each range writes unnormalised sums with their maximum and weight
// sum, and pta_attn_combine merges them in range order.
//
// The keys of the next block are asked for as soon as the products with the current ones are done, the values of the
// current block at its start: both arrive behind the cap, the mix and the softmax of the block.
#pragma once

#include "common.h"
#include "pta_kernels.h"

typedef __bf16 talk_bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 talk_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float talk_f32x4_t __attribute__((ext_vector_type(4)));
typedef float talk_f32x2_t __attribute__((ext_vector_type(2)));

union TalkFrag {
    uint4 u;
    talk_bf16x8_t v;
};

__device__ __forceinline__ uint32_t talk_pack_bf16(float lo, float hi) {
    union { talk_bf16x2_t b; uint32_t u; } c;
    c.b = __builtin_convertvector(talk_f32x2_t{lo, hi}, talk_bf16x2_t);
    return c.u;
}

#define TALK_LOG2E 1.4426950408889634f

// DT: head size / 16.  CT: heads of a wave (all of one KV head).  MAXW: the most waves a workgroup has (the
// registers a wave may use follow from it).
template <int DT, int CT, int MAXW>
__global__ __launch_bounds__(64 * MAXW) void attn_talk_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ po, float* __restrict__ pm, float* __restrict__ pl,
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    const int* __restrict__ block_table, int bt_stride, const int* __restrict__ cu_tokens,
    const int* __restrict__ seq_start, const float* __restrict__ talk, float cap, float pre_mul, int nh, int nkv,
    int window, int chunk, int split_size, int n_splits, const float* __restrict__ head_scale,
    const float* __restrict__ head_bias, int weights_kind, int heads_wg) {
    constexpr int D = DT * 16, DS = (DT + 1) / 2, CHUNKS = D / 8;
    extern __shared__ __attribute__((aligned(16))) float4 talk_tiles[];  // [2][nh][2][64], then the mix [nh][nh]
    auto lowest_key = [&](int t) {
        int lo = window > 0 ? max(0, t - window + 1) : 0;
        if (chunk > 0) lo = max(lo, t / chunk * chunk);
        return lo;
    };
    const int lane = threadIdx.x & 63, c = lane & 15, gq = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_seqs = gridDim.y / n_splits;
    const int seq = blockIdx.y % n_seqs, split = blockIdx.y / n_seqs;
    const int t0 = cu_tokens[seq], n_new = cu_tokens[seq + 1] - t0, start = seq_start[seq];
    const int tok0 = (int)(gridDim.x - 1 - blockIdx.x) * 16;  // late tokens, which see the most keys, start first
    if (tok0 >= n_new) return;
    const int g = nh / nkv, h0 = blockIdx.z * heads_wg + wave * CT, kvh = h0 / g;
    const int tok = t0 + min(tok0 + c, n_new - 1);
    const int qpos = tok0 + c < n_new ? start + tok0 + c : -1;  // -1: a column that does not exist sees no key
    const int first_pos = start + tok0, last_pos = start + min(tok0 + 15, n_new - 1);
    const int kv_len = start + n_new;
    const int lo_last = lowest_key(last_pos);
    int k_begin = lowest_key(first_pos) & ~31, k_end = last_pos + 1;
    if (n_splits > 1) {
        if (split_size > 0) {  // ranges of the context
            k_begin = max(k_begin, split * split_size);
            k_end = min(k_end, (split + 1) * split_size);
        } else {               // equal runs of this tile's blocks
            const int per = ((k_end - k_begin + 31) / 32 + n_splits - 1) / n_splits * 32;
            k_begin += split * per;
            k_end = min(k_end, k_begin + per);
        }
    }
    const int min_lim = min(first_pos + 1, k_end);  // below this key no column masks anything for being late

    if (k_begin >= k_end) {  // a range that none of the tokens sees: only its marker is written
        if (n_splits > 1 && qpos >= 0 && gq == 0) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                const long row = (long)tok * nh + h0 + ct;
                pm[row * n_splits + split] = -INFINITY;
                pl[row * n_splits + split] = 0.f;
            }
        }
        return;
    }

    TalkFrag qf[CT][DS];
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const bf16_t* qp = q + ((long)tok * nh + h0 + ct) * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int piece = ds * 4 + gq;
            qf[ct][ds].u = *reinterpret_cast<const uint4*>(qp + min(piece, CHUNKS - 1) * 8);
            if (piece >= CHUNKS) qf[ct][ds].u = zero4;  // an odd number of 16-wide tiles: the last step is half empty
        }
    }
    talk_f32x4_t oacc[DT][CT], lacc[CT];
    float m_run[CT], m_raise[CT], mul_h[CT], bias_h[CT];
    const bool sig = weights_kind == PTA_WEIGHTS_SIGMOID;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        mul_h[ct] = head_scale ? pre_mul * head_scale[h0 + ct] : pre_mul;
        bias_h[ct] = head_bias ? head_bias[h0 + ct] * TALK_LOG2E : 0.f;
        m_run[ct] = -INFINITY;
        m_raise[ct] = -INFINITY;
        lacc[ct] = talk_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) oacc[dt][ct] = talk_f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    TalkFrag ones;
    ones.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);
    const int* bt = block_table + (long)seq * bt_stride;
    const float cap2 = -2.0f * cap;
    float* mix_s = reinterpret_cast<float*>(talk_tiles + (size_t)nh * 256);
    if (talk) {
        for (int i = threadIdx.x; i < nh * nh; i += blockDim.x) mix_s[i] = talk[i];
        // (read only behind the first block's barrier)
    }
    const float* mix_row = mix_s + h0 * nh;

    // key rows: tile tt, row r holds key 8*(r/4) + 4*tt + r%4 of the block, so that a lane's eight scores are
    // those of the eight consecutive keys 8*gq .. 8*gq+7, which is what the second product's operand wants
    TalkFrag kf[2][DS];
    auto load_keys = [&](int kb) {
        const long page = ((long)bt[kb >> 6] * nkv + kvh) * (long)(PTA_PAGE * D);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            const bf16_t* kp = k_pool + page + (long)((kb & 63) + 8 * (c >> 2) + 4 * tt + (c & 3)) * D;
#pragma unroll
            for (int ds = 0; ds < DS; ++ds)
                kf[tt][ds].u = *reinterpret_cast<const uint4*>(kp + min(ds * 4 + gq, CHUNKS - 1) * 8);
        }
    };
    const int kb_last = (kv_len - 1) & ~31;  // the last block that has a page
    // (not where sixteen waves of large heads leave a wave no registers for it)
    constexpr bool AHEAD = MAXW <= 8 || DT <= 4;
    if constexpr (AHEAD) load_keys(k_begin);

    int it = 0;
    for (int kb = k_begin; kb < k_end; kb += 32, ++it) {
        const long page = ((long)bt[kb >> 6] * nkv + kvh) * (long)(PTA_PAGE * D);
        const int in_page = kb & 63;
        TalkFrag vf[DT];
        if constexpr (!AHEAD) load_keys(kb);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
            vf[dt].u = *reinterpret_cast<const uint4*>(v_pool + page + (long)(dt * 16 + c) * PTA_PAGE + in_page + gq * 8);

        talk_f32x4_t s[2][CT];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                talk_f32x4_t acc = talk_f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < DS; ++ds)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[tt][ds].v, qf[ct][ds].v, acc, 0, 0, 0);
                s[tt][ct] = acc;
            }
        if constexpr (AHEAD) load_keys(min(kb + 32, kb_last));  // the next block's (the last one's again behind it)
#pragma unroll
        for (int tt = 0; tt < 2; ++tt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    float x = s[tt][ct][e] * mul_h[ct];
                    // cap * tanh(z) = cap - 2 cap / (1 + e^(2z)); pre_mul carries 2 scale log2(e) / cap
                    if (cap > 0.f) x = __builtin_fmaf(cap2, __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x)), cap);
                    s[tt][ct][e] = x;
                }

        if (talk) {
            float4* tiles = talk_tiles + (size_t)(it & 1) * nh * 128;
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
#pragma unroll
                for (int tt = 0; tt < 2; ++tt)
                    tiles[((h0 + ct) * 2 + tt) * 64 + lane] = make_float4(s[tt][ct][0], s[tt][ct][1], s[tt][ct][2], s[tt][ct][3]);
            __syncthreads();
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                s[0][ct] = talk_f32x4_t{0.f, 0.f, 0.f, 0.f};
                s[1][ct] = talk_f32x4_t{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll 4
            for (int h = 0; h < nh; ++h) {
                const float4 a0 = tiles[(h * 2) * 64 + lane], a1 = tiles[(h * 2 + 1) * 64 + lane];
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) {
                    const float t = mix_row[ct * nh + h];
                    s[0][ct][0] = __builtin_fmaf(t, a0.x, s[0][ct][0]); s[0][ct][1] = __builtin_fmaf(t, a0.y, s[0][ct][1]);
                    s[0][ct][2] = __builtin_fmaf(t, a0.z, s[0][ct][2]); s[0][ct][3] = __builtin_fmaf(t, a0.w, s[0][ct][3]);
                    s[1][ct][0] = __builtin_fmaf(t, a1.x, s[1][ct][0]); s[1][ct][1] = __builtin_fmaf(t, a1.y, s[1][ct][1]);
                    s[1][ct][2] = __builtin_fmaf(t, a1.z, s[1][ct][2]); s[1][ct][3] = __builtin_fmaf(t, a1.w, s[1][ct][3]);
                }
            }
        }

        // positions past the sequence's end were never written; whatever lies there must not reach the sums, not
        // even with weight zero
        if (kb + 32 > kv_len) {
            const int kbase = kb + gq * 8;
            uint32_t mk[4];
#pragma unroll
            for (int w = 0; w < 4; ++w)
                mk[w] = (kbase + 2 * w < kv_len ? 0x0000ffffu : 0u) | (kbase + 2 * w + 1 < kv_len ? 0xffff0000u : 0u);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                vf[dt].u.x &= mk[0]; vf[dt].u.y &= mk[1]; vf[dt].u.z &= mk[2]; vf[dt].u.w &= mk[3];
            }
        }

        const bool interior = kb + 32 <= min_lim && kb >= lo_last;
        TalkFrag pf[CT];
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (!interior) {
                const int lim = min(qpos + 1, k_end);
                const int lo = lowest_key(max(qpos, 0));
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (kb + 8 * gq + j >= lim || kb + 8 * gq + j < lo) s[j >> 2][ct][j & 3] = -INFINITY;
            }
            if (sig) {  // 1 / (1 + 2^(-(s + bias) log2 e)); a key that is not seen has s = -inf and the weight 0
                float p[8];
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    p[j] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-__builtin_fmaf(s[j >> 2][ct][j & 3], TALK_LOG2E, bias_h[ct])));
                pf[ct].u = make_uint4(talk_pack_bf16(p[0], p[1]), talk_pack_bf16(p[2], p[3]), talk_pack_bf16(p[4], p[5]),
                                      talk_pack_bf16(p[6], p[7]));
                continue;
            }
            float mx = fmaxf(fmaxf(fmaxf(s[0][ct][0], s[0][ct][1]), fmaxf(s[0][ct][2], s[0][ct][3])),
                             fmaxf(fmaxf(s[1][ct][0], s[1][ct][1]), fmaxf(s[1][ct][2], s[1][ct][3])));
            // The running maximum is a reference point for the exponentials, shared by the four lanes of a column;
            // it is brought up (and what was summed rescaled) only when a score lies more than 2^8 above it
            if (__any(mx > m_raise[ct])) {
                float m = mx * TALK_LOG2E;
                m = fmaxf(m, __shfl_xor(m, 16, 64));
                m = fmaxf(m, __shfl_xor(m, 32, 64));
                const float m_new = fmaxf(m_run[ct], m);
                const float corr = __builtin_amdgcn_exp2f(m_run[ct] - (m_new == -INFINITY ? 0.f : m_new));
                lacc[ct][0] *= corr;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) {
                    oacc[dt][ct][0] *= corr; oacc[dt][ct][1] *= corr; oacc[dt][ct][2] *= corr; oacc[dt][ct][3] *= corr;
                }
                m_run[ct] = m_new;
                m_raise[ct] = (m_new + 8.0f) * (1.0f / TALK_LOG2E);
            }
            const float m_use = m_run[ct] == -INFINITY ? 0.f : m_run[ct];
            float p[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[j >> 2][ct][j & 3], TALK_LOG2E, -m_use));
            pf[ct].u = make_uint4(talk_pack_bf16(p[0], p[1]), talk_pack_bf16(p[2], p[3]), talk_pack_bf16(p[4], p[5]),
                                  talk_pack_bf16(p[6], p[7]));
        }
        if (!sig) {
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                lacc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pf[ct].v, lacc[ct], 0, 0, 0);
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                oacc[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt].v, pf[ct].v, oacc[dt][ct], 0, 0, 0);
    }

#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        if (qpos < 0) continue;
        // (unnormalised weights: the ranges' sums are added as they are, which the merge does when every range that has
        // keys says maximum 0 and exactly one of them, the one that holds the token's own position, weight sum 1)
        const float l = sig ? ((n_splits == 1 || (qpos >= k_begin && qpos < k_end)) ? 1.f : 0.f) : lacc[ct][0];
        const long row = (long)tok * nh + h0 + ct;
        if (n_splits == 1) {
            const float inv = 1.0f / l;
            bf16_t* o = out + row * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                uint2 w;
                w.x = talk_pack_bf16(oacc[dt][ct][0] * inv, oacc[dt][ct][1] * inv);
                w.y = talk_pack_bf16(oacc[dt][ct][2] * inv, oacc[dt][ct][3] * inv);
                *reinterpret_cast<uint2*>(o + dt * 16 + gq * 4) = w;
            }
        } else {
            float* o = po + (row * n_splits + split) * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                *reinterpret_cast<float4*>(o + dt * 16 + gq * 4) =
                    make_float4(oacc[dt][ct][0], oacc[dt][ct][1], oacc[dt][ct][2], oacc[dt][ct][3]);
            if (gq == 0) {
                pm[row * n_splits + split] = sig ? 0.f : m_run[ct];
                pl[row * n_splits + split] = l;
            }
        }
    }
}

struct TalkLaunch {
    bf16_t* out; float *po, *pm, *pl;
    const bf16_t *q, *k_pool, *v_pool;
    const int* block_table; int bt_stride;
    const int *cu_tokens, *seq_start; const float* talk; float cap, pre_mul;
    int n_seqs, max_new, nh, nkv, window, chunk, split_size, n_splits;
    hipStream_t s;
    const float *head_scale, *head_bias; int weights_kind, heads_wg;
};

// heads that one wave may hold at this head size (the registers of the sums set it)
constexpr int talk_max_heads(int dt) { return dt <= 4 ? 4 : 2; }

template <int DT, int CT, int MAXW>
static void talk_launch_one(const TalkLaunch& a) {
    auto kern = attn_talk_mfma_kernel<DT, CT, MAXW>;
    const size_t lds = a.talk ? (size_t)a.nh * 4096 + (size_t)a.nh * a.nh * 4 : 0;
    if (lds > 64 * 1024) {  // more than a launch may ask for unless the kernel has been told, once per device
        static bool told[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
        if (!told[dev]) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, 136 * 1024);
            told[dev] = true;
        }
    }
    const dim3 grid((a.max_new + 15) / 16, a.n_seqs * a.n_splits, a.nh / a.heads_wg);
    hipLaunchKernelGGL(kern, grid, dim3(64 * (a.heads_wg / CT)), lds, a.s, a.out, a.po, a.pm, a.pl, a.q, a.k_pool, a.v_pool,
                       a.block_table, a.bt_stride, a.cu_tokens, a.seq_start, a.talk, a.cap, a.pre_mul, a.nh, a.nkv, a.window,
                       a.chunk, a.split_size, a.n_splits, a.head_scale, a.head_bias, a.weights_kind, a.heads_wg);
}

// What pta_attn_talk_mfma launches for heads of DT x 16 elements with `ct` heads a wave; every head size is a
// translation unit of its own (attn_talk_mfma_dt*.hip).  false: that combination is not built.
template <int DT>
bool talk_launch_head(const TalkLaunch& a, int ct) {
    const int waves = a.heads_wg / ct;
#define TALK_CASE(CT_)                                          \
    if (ct == CT_) {                                            \
        if (waves <= 8) talk_launch_one<DT, CT_, 8>(a);         \
        else talk_launch_one<DT, CT_, 16>(a);                   \
        return true;                                            \
    }
    TALK_CASE(1)
    TALK_CASE(2)
    if constexpr (talk_max_heads(DT) >= 4) { TALK_CASE(4) }
#undef TALK_CASE
    return false;
}
