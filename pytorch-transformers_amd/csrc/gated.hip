// Element-wise gates between two matrix products.
//
// pta_gated_heads:  out[m, h * dv + e] = n(x)[m, h, e] * sigmoid(g[m, h * dv + e]), where x holds heads of dv elements
//                   in frames x_head apart (an attention result whose frames are wider than its values), and n is
//                   the identity or an RMS norm over the whole row of heads * dv elements with a weight.  With
//                   g_per_head the gate is one number a head: sigmoid(g[m, h]).
// pta_xielu:        out[m, f] = z > 0 ? ap * z^2 + z / 2 : an * (e^z - 1 - z) + z / 2 with ap = softplus(act[0]) and
//                   an = 1/2 + softplus(act[1]), act two learned numbers held in 32-bit.
// pta_glu:          out[m, f] = act(gate[m, f], up[m, f]) for a feed-forward with a gate:
//                   PTA_GLU_SILU        silu(gate) * up
//                   PTA_GLU_CLAMPED     g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1)
// Arithmetic in 32-bit, results in the compute type.
#include "common.h"
#include "pta_kernels.h"

#include <algorithm>

template <typename T, typename TX>
__global__ __launch_bounds__(1024) void gated_heads_kernel(T* __restrict__ out, const TX* __restrict__ x, long x_ld,
                                                          int x_head, const T* __restrict__ g, long g_ld,
                                                          const float* __restrict__ w, float eps, int heads, int dv,
                                                          int g_per_head) {
    __shared__ float red[16];
    const int m = blockIdx.x, N = heads * dv;
    const TX* xr = x + (long)m * x_ld;
    float inv = 1.f;
    if (w) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < N; i += blockDim.x) {
            const float v = Io<TX>::ld(xr + (long)(i / dv) * x_head + i % dv);
            ss += v * v;
        }
        inv = rsqrtf(block_sum(ss, red) / (float)N + eps);
    }
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        float v = Io<TX>::ld(xr + (long)(i / dv) * x_head + i % dv);
        if (w) v = v * inv * w[i];
        const float gate = 1.0f / (1.0f + expf(-Io<T>::ld(g + (long)m * g_ld + (g_per_head ? i / dv : i))));
        Io<T>::st(out + (long)m * N + i, v * gate);
    }
}

// x: 32-bit (x_f32) or the compute type; g and out in the compute type
extern "C" int pta_gated_heads(void* out, const void* x, int x_f32, long x_ld, int x_head, const void* g, long g_ld,
                               const float* w, float eps, int M, int heads, int dv, int g_per_head, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && heads > 0 && dv > 0, "gated_heads: sizes must be positive");
    PTA_REQUIRE(out && x && g, "gated_heads: null pointer");
    PTA_REQUIRE(x_head >= dv && x_ld >= (long)(heads - 1) * x_head + dv && g_ld >= (long)heads * (g_per_head ? 1 : dv),
                "gated_heads: rows or frames lie closer together than they are long");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "gated_heads: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(M), block(std::min(1024, std::max(64, (heads * dv / 4 + 63) / 64 * 64)));
    if (dtype == PTA_F32)
        hipLaunchKernelGGL((gated_heads_kernel<float, float>), grid, block, 0, s, (float*)out, (const float*)x, x_ld, x_head,
                           (const float*)g, g_ld, w, eps, heads, dv, g_per_head);
    else if (x_f32)
        hipLaunchKernelGGL((gated_heads_kernel<bf16_t, float>), grid, block, 0, s, (bf16_t*)out, (const float*)x, x_ld, x_head,
                           (const bf16_t*)g, g_ld, w, eps, heads, dv, g_per_head);
    else
        hipLaunchKernelGGL((gated_heads_kernel<bf16_t, bf16_t>), grid, block, 0, s, (bf16_t*)out, (const bf16_t*)x, x_ld,
                           x_head, (const bf16_t*)g, g_ld, w, eps, heads, dv, g_per_head);
    return pta_check_launch("gated_heads");
}

template <typename T>
__global__ void glu_kernel(T* __restrict__ out, const T* __restrict__ gate, const T* __restrict__ up, long in_ld, int F,
                           long n, int kind, float alpha, float limit) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long m = i / F, f = i - m * F;
    float g = Io<T>::ld(gate + m * in_ld + f), u = Io<T>::ld(up + m * in_ld + f);
    float y;
    if (kind == PTA_GLU_CLAMPED) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        y = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    } else {
        y = g / (1.0f + expf(-g)) * u;
    }
    Io<T>::st(out + i, y);
}

// gate, up: [M, F] with rows in_ld apart (the two halves of one product's rows); out [M, F] dense
extern "C" int pta_glu(void* out, const void* gate, const void* up, long in_ld, int M, int F, int kind, float alpha,
                       float limit, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && F > 0 && out && gate && up && in_ld >= F, "glu: sizes must be positive and pointers given");
    PTA_REQUIRE(kind == PTA_GLU_SILU || kind == PTA_GLU_CLAMPED, "glu: kind %d is not built", kind);
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "glu: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const long n = (long)M * F;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(glu_kernel<float>, grid, dim3(256), 0, s, (float*)out, (const float*)gate, (const float*)up, in_ld, F, n, kind, alpha, limit);
    else
        hipLaunchKernelGGL(glu_kernel<bf16_t>, grid, dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)gate, (const bf16_t*)up, in_ld, F, n, kind, alpha, limit);
    return pta_check_launch("glu");
}

// z: [M, F] with rows z_ld apart; out [M, F] dense.  softplus in 32-bit (the identity beyond 20, where 1 + e^v rounds to e^v).
__device__ __forceinline__ float softplus_f32(float v) { return v > 20.f ? v : log1pf(expf(v)); }

template <typename T>
__global__ void xielu_kernel(T* __restrict__ out, const T* __restrict__ z, long z_ld, int F, long n,
                             const float* __restrict__ act) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const long m = i / F, f = i - m * F;
    Io<T>::st(out + i, xielu_value(Io<T>::ld(z + m * z_ld + f), softplus_f32(act[0]), 0.5f + softplus_f32(act[1])));
}

// bfloat16 rows of a multiple of eight elements at sixteen-byte addresses: eight elements a thread
__global__ void xielu_bf16x8_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ z, long z_ld, int F8, long n8,
                                    const float* __restrict__ act) {
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    const long m = i / F8, f = (i - m * F8) * 8;
    const float ap = softplus_f32(act[0]), an = 0.5f + softplus_f32(act[1]);
    float v[8];
    unpack8(*reinterpret_cast<const uint4*>(z + m * z_ld + f), v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = xielu_value(v[e], ap, an);
    *reinterpret_cast<uint4*>(out + m * (long)F8 * 8 + f) = pack8(v);
}

extern "C" int pta_xielu(void* out, const void* z, long z_ld, int M, int F, const float* act, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && F > 0 && out && z && act && z_ld >= F, "xielu: sizes must be positive and pointers given");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "xielu: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const long n = (long)M * F;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(xielu_kernel<float>, grid, dim3(256), 0, s, (float*)out, (const float*)z, z_ld, F, n, act);
    else if (F % 8 == 0 && z_ld % 8 == 0 && ((uintptr_t)z % 16) == 0 && ((uintptr_t)out % 16) == 0)
        hipLaunchKernelGGL(xielu_bf16x8_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s, (bf16_t*)out,
                           (const bf16_t*)z, z_ld, F / 8, n / 8, act);
    else
        hipLaunchKernelGGL(xielu_kernel<bf16_t>, grid, dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)z, z_ld, F, n, act);
    return pta_check_launch("xielu");
}

// PolyNorm (see pta_kernels.h): one workgroup per row, the three mean squares in one pass, the row read again for the
// output.  Sums are 32-bit, in an order that depends on the row's length alone.
template <typename T>
__global__ __launch_bounds__(256) void polynorm_kernel(T* __restrict__ out, const T* __restrict__ z, long z_ld,
                                                       const float* __restrict__ coef, float eps, int F) {
    __shared__ float red[16];
    const T* zr = z + (long)blockIdx.x * z_ld;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < F; i += blockDim.x) {
        const float v = Io<T>::ld(zr + i), v2 = v * v;
        s1 += v2;
        s2 += v2 * v2;
        s3 += v2 * v2 * v2;
    }
    const float inv_f = 1.0f / (float)F;
    const float r1 = coef[0] / sqrtf(block_sum(s1, red) * inv_f + eps);
    const float r2 = coef[1] / sqrtf(block_sum(s2, red) * inv_f + eps);
    const float r3 = coef[2] / sqrtf(block_sum(s3, red) * inv_f + eps);
    const float e = coef[3];
    T* orow = out + (long)blockIdx.x * F;
    for (int i = threadIdx.x; i < F; i += blockDim.x) {
        const float v = Io<T>::ld(zr + i), v2 = v * v;
        Io<T>::st(orow + i, r1 * v + r2 * v2 + r3 * (v2 * v) + e);
    }
}

// The same for bfloat16 rows whose length is a multiple of eight and that start at multiples of 16 bytes: eight
// elements a load, long rows on 1,024 threads.
__device__ __forceinline__ void polynorm_unpack(const uint4& u, float (&v)[8]) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(w[j] << 16);
        v[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
    }
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void polynorm_vec_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ z,
                                                               long z_ld, const float* __restrict__ coef, float eps, int F) {
    __shared__ float red[16];
    const uint4* zr = reinterpret_cast<const uint4*>(z + (long)blockIdx.x * z_ld);
    const int n = F / 8;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < n; i += THREADS) {
        float v[8];
        polynorm_unpack(zr[i], v);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float v2 = v[j] * v[j];
            s1 += v2;
            s2 += v2 * v2;
            s3 += v2 * v2 * v2;
        }
    }
    const float inv_f = 1.0f / (float)F;
    const float r1 = coef[0] / sqrtf(block_sum(s1, red) * inv_f + eps);
    const float r2 = coef[1] / sqrtf(block_sum(s2, red) * inv_f + eps);
    const float r3 = coef[2] / sqrtf(block_sum(s3, red) * inv_f + eps);
    const float e = coef[3];
    uint4* orow = reinterpret_cast<uint4*>(out + (long)blockIdx.x * F);
    for (int i = threadIdx.x; i < n; i += THREADS) {
        float v[8];
        polynorm_unpack(zr[i], v);
        bf16_t r[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float v2 = v[j] * v[j];
            r[j] = f32_to_bf16_bits(r1 * v[j] + r2 * v2 + r3 * (v2 * v[j]) + e);
        }
        orow[i] = *reinterpret_cast<const uint4*>(r);
    }
}

extern "C" int pta_polynorm(void* out, const void* z, long z_ld, const float* coef, float eps, int M, int F, int dtype,
                            void* stream) {
    PTA_REQUIRE(M > 0 && F > 0 && out && z && coef && z_ld >= F, "polynorm: sizes must be positive and pointers given");
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(polynorm_kernel<float>, dim3(M), dim3(256), 0, s, (float*)out, (const float*)z, z_ld, coef, eps, F);
    else if (dtype == PTA_BF16 && F % 8 == 0 && z_ld % 8 == 0 && (uintptr_t)z % 16 == 0 && (uintptr_t)out % 16 == 0) {
        // (the threads of a row follow from its length alone, so the sums' order does not depend on the batch)
        if (F >= 8192)
            hipLaunchKernelGGL(polynorm_vec_kernel<1024>, dim3(M), dim3(1024), 0, s, (bf16_t*)out, (const bf16_t*)z, z_ld, coef, eps, F);
        else
            hipLaunchKernelGGL(polynorm_vec_kernel<256>, dim3(M), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)z, z_ld, coef, eps, F);
    } else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(polynorm_kernel<bf16_t>, dim3(M), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)z, z_ld, coef, eps, F);
    else
        return pta_fail("polynorm: unknown dtype %d", dtype);
    return pta_check_launch("polynorm");
}
