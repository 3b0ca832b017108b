// LayerNorm (mean, biased variance, weight and bias) around a residual stream that is held in 32-bit whatever the
// model's compute type.  One launch does what stands between two sublayers of a block that norms a sublayer's
// output as well as its input:
//
//   s = x                                  the stream (32-bit), if given
//   s += mult * (LN(y) * wy + by)          a sublayer's output y (compute type) normed, scaled and added, if given
//   s += add                               another 32-bit tensor of the stream's shape (rows of its own), if given
//   s += vec                               one 32-bit vector for every row, if given
//   out_wide = s                           if wanted
//   out_narrow = LN(s) * w + b             in the compute type, if w is given; without w, s itself in the compute type
//
// `rows` gathers: output row m is made of input row rows[m] (the final norm on the wanted rows alone).
// One workgroup per row; a thread keeps its VPT elements in registers over all passes; every sum over a row is taken
// in 32-bit in an order that depends on the row's length alone.
#include "common.h"
#include "pta_kernels.h"

template <typename T, int VPT>
__global__ __launch_bounds__(256) void layernorm_stream_kernel(T* __restrict__ out_narrow, float* __restrict__ out_wide,
                                                               const float* __restrict__ x, const T* __restrict__ y, long y_ld,
                                                               const float* __restrict__ wy, const float* __restrict__ by,
                                                               float mult, const float* __restrict__ add,
                                                               const float* __restrict__ vec, const int* __restrict__ rows,
                                                               const float* __restrict__ w, const float* __restrict__ b,
                                                               float eps, int H) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const long src = rows ? rows[m] : m;
    const float inv_h = 1.0f / (float)H;
    float s[VPT], yv[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {  // every load of the first pass asked for at once
        const int i = threadIdx.x + k * blockDim.x;
        s[k] = (x && i < H) ? x[src * H + i] : 0.f;
        yv[k] = (y && i < H) ? Io<T>::ld(y + src * y_ld + i) : 0.f;
    }
    if (y) {
        float wv[VPT], bv[VPT];
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            wv[k] = i < H ? wy[i] : 0.f;
            bv[k] = i < H ? by[i] : 0.f;
        }
        float t = 0.f;
#pragma unroll
        for (int k = 0; k < VPT; ++k) t += yv[k];
        const float mean = block_sum(t, red) * inv_h;
        t = 0.f;
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            const float dlt = i < H ? yv[k] - mean : 0.f;
            t += dlt * dlt;
        }
        const float inv = 1.0f / sqrtf(block_sum(t, red) * inv_h + eps);
#pragma unroll
        for (int k = 0; k < VPT; ++k) s[k] += mult * ((yv[k] - mean) * inv * wv[k] + bv[k]);
    }
    if (add) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            if (i < H) s[k] += add[src * H + i];
        }
    }
    if (vec) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            if (i < H) s[k] += vec[i];
        }
    }
    if (out_wide) {
#pragma unroll
        for (int k = 0; k < VPT; ++k) {
            const int i = threadIdx.x + k * blockDim.x;
            if (i < H) out_wide[(long)m * H + i] = s[k];
        }
    }
    if (!w) {
        if (out_narrow) {
#pragma unroll
            for (int k = 0; k < VPT; ++k) {
                const int i = threadIdx.x + k * blockDim.x;
                if (i < H) Io<T>::st(out_narrow + (long)m * H + i, s[k]);
            }
        }
        return;
    }
    float wv[VPT], bv[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + k * blockDim.x;
        wv[k] = i < H ? w[i] : 0.f;
        bv[k] = i < H ? b[i] : 0.f;
    }
    float t = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + k * blockDim.x;
        t += i < H ? s[k] : 0.f;
    }
    const float mean = block_sum(t, red) * inv_h;
    t = 0.f;
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + k * blockDim.x;
        const float dlt = i < H ? s[k] - mean : 0.f;
        t += dlt * dlt;
    }
    const float inv = 1.0f / sqrtf(block_sum(t, red) * inv_h + eps);
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int i = threadIdx.x + k * blockDim.x;
        if (i < H) Io<T>::st(out_narrow + (long)m * H + i, (s[k] - mean) * inv * wv[k] + bv[k]);
    }
}

template <typename T>
static int launch_ln_stream(void* out_narrow, float* out_wide, const float* x, const void* y, long y_ld, const float* wy,
                            const float* by, float mult, const float* add, const float* vec, const int* rows, const float* w,
                            const float* b, float eps, int M, int H, hipStream_t s) {
    // the block's size follows from the row's length alone
    const int threads = H <= 64 ? 64 : H <= 128 ? 128 : 256;
    const int vpt = (H + threads - 1) / threads;
#define PTA_LN_STREAM(V)                                                                                                    \
    hipLaunchKernelGGL((layernorm_stream_kernel<T, V>), dim3(M), dim3(threads), 0, s, (T*)out_narrow, out_wide, x, (const T*)y, \
                       y_ld, wy, by, mult, add, vec, rows, w, b, eps, H)
    if (vpt <= 1) PTA_LN_STREAM(1);
    else if (vpt <= 2) PTA_LN_STREAM(2);
    else if (vpt <= 4) PTA_LN_STREAM(4);
    else if (vpt <= 8) PTA_LN_STREAM(8);
    else if (vpt <= 16) PTA_LN_STREAM(16);
    else if (vpt <= 32) PTA_LN_STREAM(32);
    else return pta_fail("layernorm_stream: rows of %d features are more than the 8192 the kernel holds", H);
#undef PTA_LN_STREAM
    return pta_check_launch("layernorm_stream");
}

extern "C" int pta_layernorm_stream(void* out_narrow, float* out_wide, const float* x, const void* y, long y_ld,
                                    const float* wy, const float* by, float mult, const float* add, const float* vec,
                                    const int* rows, const float* w, const float* b, float eps, int M, int H, int dtype,
                                    void* stream) {
    PTA_REQUIRE(M > 0 && H > 0, "layernorm_stream: sizes must be positive (M=%d H=%d)", M, H);
    PTA_REQUIRE(x || y, "layernorm_stream: neither a stream nor a sublayer's output given");
    PTA_REQUIRE(!y || (wy && by && y_ld >= H), "layernorm_stream: a sublayer's output needs its norm's weight and bias");
    PTA_REQUIRE((w != nullptr) == (b != nullptr), "layernorm_stream: weight and bias come together");
    PTA_REQUIRE(!w || out_narrow, "layernorm_stream: a norm of the stream needs a place for its output");
    PTA_REQUIRE(out_narrow || out_wide, "layernorm_stream: nothing to write");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        return launch_ln_stream<float>(out_narrow, out_wide, x, y, y_ld, wy, by, mult, add, vec, rows, w, b, eps, M, H, s);
    if (dtype == PTA_BF16)
        return launch_ln_stream<bf16_t>(out_narrow, out_wide, x, y, y_ld, wy, by, mult, add, vec, rows, w, b, eps, M, H, s);
    return pta_fail("layernorm_stream: unknown dtype %d", dtype);
}
