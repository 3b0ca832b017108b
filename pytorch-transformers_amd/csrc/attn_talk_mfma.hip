// The entry point of the attention with capped, mixed scores on the matrix cores; the kernel and its launchers are in
// attn_talk_mfma_impl.h, instantiated per head size in attn_talk_mfma_dt*.hip.
#include "attn_talk_mfma_impl.h"

#include <stdlib.h>

#include <algorithm>

#define PTA_TALK_HEAD(DT_) extern template bool talk_launch_head<DT_>(const TalkLaunch&, int);
PTA_TALK_HEAD(1) PTA_TALK_HEAD(2) PTA_TALK_HEAD(3) PTA_TALK_HEAD(4) PTA_TALK_HEAD(5) PTA_TALK_HEAD(6) PTA_TALK_HEAD(7)
PTA_TALK_HEAD(8)
#undef PTA_TALK_HEAD

// heads a wave holds: as many as the head size allows, all of one KV head, with at most sixteen waves; 0: none fits.
// heads_wg: the heads of a workgroup: all of them where the scores are mixed over the heads; without a mix the heads
// of one KV head (or sixteen waves' worth of them), so that a token's heads spread over several workgroups.
static int talk_heads_per_wave(int nh, int nkv, int d, bool mixed, int* heads_wg) {
    if (nh <= 0 || nkv <= 0 || nh % nkv || d % 16 || d < 16 || d > 128) return 0;
    if (mixed && (size_t)nh * 4096 > 128 * 1024) return 0;  // the heads' tiles of two blocks of keys in LDS
    const int g = nh / nkv;
    // PTA_TALK_HEADS: fewer heads a wave than the head size allows, for measurements (16 heads of 128 with a head a
    // wave on sixteen waves: 156 us a layer of 2,048 tokens against 107 with two heads a wave on eight; every wave reads
    // all heads' tiles, so twice the waves read twice as much from LDS)
    static const int most_env = getenv("PTA_TALK_HEADS") ? atoi(getenv("PTA_TALK_HEADS")) : 0;
    const int most = most_env > 0 ? std::min(most_env, talk_max_heads(d / 16)) : talk_max_heads(d / 16);
    for (int ct = most; ct >= 1; ct /= 2) {
        if (g % ct) continue;
        if (mixed) {
            if (nh / ct > 16) continue;
            if (heads_wg) *heads_wg = nh;
            return ct;
        }
        int waves = g / ct;  // of one KV head; more than sixteen are cut into equal parts
        while (waves > 16) {
            int f = 2;
            while (waves % f) ++f;
            waves /= f;
        }
        if (heads_wg) *heads_wg = waves * ct;
        return ct;
    }
    return 0;
}

// Into how many runs a prompt launch cuts every tile's keys: the tiles alone should not leave compute units idle, a
// run is at least four blocks of keys, and at most four partial results a row are written and merged.
extern "C" int pta_attn_talk_prompt_ranges(int tiles, int keys_seen) {
    const int units = pta_compute_units();
    if (tiles <= 0 || tiles >= units) return 1;
    return std::max(1, std::min({4, units / tiles, keys_seen / 128}));
}

// mixed: whether the scores are mixed over the heads (then a workgroup holds all heads of its tokens)
extern "C" int pta_attn_talk_mfma_supported(int nh, int nkv, int d, int mixed) {
    return talk_heads_per_wave(nh, nkv, d, mixed != 0, nullptr) > 0;
}
// workgroups that share a token's heads in a launch
extern "C" int pta_attn_talk_mfma_workgroups(int nh, int nkv, int d, int mixed) {
    int heads_wg = 0;
    return talk_heads_per_wave(nh, nkv, d, mixed != 0, &heads_wg) > 0 ? nh / heads_wg : 0;
}

extern "C" int pta_attn_talk_mfma(void* out, const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                                  int bt_stride, const int* cu_tokens, const int* seq_start, const float* talk, float softcap,
                                  int n_seqs, int max_new, int M, int nh, int nkv, int d, float scale, int window, int chunk,
                                  int split_size, int n_splits, float* po, float* pm, float* pl, const float* head_scale,
                                  const float* head_bias, int weights_kind, void* stream) {
    PTA_REQUIRE(weights_kind == PTA_WEIGHTS_SOFTMAX || weights_kind == PTA_WEIGHTS_SIGMOID, "attn_talk_mfma: weights of kind %d are not built", weights_kind);
    PTA_REQUIRE(n_seqs > 0 && max_new > 0 && M > 0, "attn_talk_mfma: sizes must be positive");
    int heads_wg = 0;
    const int ct = talk_heads_per_wave(nh, nkv, d, talk != nullptr, &heads_wg);
    PTA_REQUIRE(ct > 0, "attn_talk_mfma: %d heads on %d KV heads of size %d are not built (sizes 16..128 in steps of 16, "
                "at most 32 heads, at most 16 groups of heads that fit a wave)", nh, nkv, d);
    PTA_REQUIRE(window >= 0 && chunk >= 0 && softcap >= 0.f, "attn_talk_mfma: window, chunk and softcap are 0 (none) or positive");
    PTA_REQUIRE(n_splits >= 1 && n_splits <= 1024, "attn_talk_mfma: n_splits must be 1..1024, got %d", n_splits);
    PTA_REQUIRE(n_splits == 1 || (split_size >= 0 && split_size % 64 == 0 && po && pm && pl),
                "attn_talk_mfma: ranges of keys have a size that is a multiple of 64 (0: equal runs of every tile's "
                "blocks) and buffers for the partial results");
    PTA_REQUIRE((long)n_seqs * n_splits <= 65535, "attn_talk_mfma: too many sequences x ranges for one launch");
    PTA_REQUIRE(out && q && k_pool && v_pool && block_table && cu_tokens && seq_start, "attn_talk_mfma: null pointer");
    PTA_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 && ((uintptr_t)v_pool % 16) == 0 &&
                    ((uintptr_t)out % 8) == 0, "attn_talk_mfma: pointers must be 16-byte aligned");
    // cap * tanh(s scale / cap) is evaluated as cap - 2 cap / (1 + 2^(s pre_mul))
    const float pre_mul = softcap > 0.f ? 2.0f * scale * TALK_LOG2E / softcap : scale;
    const TalkLaunch a{(bf16_t*)out, po, pm, pl, (const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_table,
                       bt_stride, cu_tokens, seq_start, talk, softcap, pre_mul, n_seqs, max_new, nh, nkv, window, chunk,
                       split_size, n_splits, (hipStream_t)stream, head_scale, head_bias, weights_kind, heads_wg};
    bool built = false;
    switch (d / 16) {
#define PTA_TALK_CASE(DT_) case DT_: built = talk_launch_head<DT_>(a, ct); break;
        PTA_TALK_CASE(1) PTA_TALK_CASE(2) PTA_TALK_CASE(3) PTA_TALK_CASE(4) PTA_TALK_CASE(5) PTA_TALK_CASE(6)
        PTA_TALK_CASE(7) PTA_TALK_CASE(8)
#undef PTA_TALK_CASE
    }
    if (!built) return pta_fail("attn_talk_mfma: no kernel for %d heads a wave at head size %d", ct, d);
    int rc = pta_check_launch("attn_talk_mfma");
    if (rc || n_splits == 1) return rc;
    return pta_attn_combine(out, po, pm, pl, (long)M * nh, d, n_splits, stream);
}
