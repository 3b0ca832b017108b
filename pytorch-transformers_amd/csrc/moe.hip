// A feed-forward of routed experts.
//
//   z = W_r h (32-bit); s = score(z) (sigmoid, or softmax over the experts); the `top` largest s are taken;
//   weights = s / (sum of the taken s + 1e-20) * scale   (or the taken s times scale, unnormalised);
//   out = sum over the taken experts e of weight_e * D_e (act(G_e h) * (U_e h))
//   (z may have a bias added; in place of act(g) * u an expert may have the clamped gate of PtaGate, pta_kernels.h;
//    an expert without a gate is D_e act(U_e h), its matrices stacked as up [E, F, H]; with groups the experts form
//    `groups` equal runs of neighbours, a run's score is its largest s, and only experts of the `keep` best runs can
//    be taken; the router's launch can also form sigmoid(X h) for a few more 32-bit rows X, e.g. the gate of an expert
//    that every token uses, whose output the launch that sums the taken experts adds times that gate)
//
// Expert matrices are held stacked: gate_up [E, 2F, H] (an expert's gate rows, then its up rows) and down [E, H, F].
//
// pta_moe_route     one workgroup per token: scores, the taken experts and their weights
// pta_moe_up        per (token, taken expert): act(G h) * (U h), a wave per few rows of the expert, H walked by lanes
// pta_moe_down      per token: the weighted sum of the taken experts' down products, in the order they were taken
// These three read an expert's matrices once per (token, expert): right for steps of few tokens, whose time is the
// bytes of the experts they touch.  Steps of many tokens sort the (token, expert) pairs by expert and run tiles of
// rows of one expert on the matrix cores (pta_moe_sort, pta_moe_grouped_*), so that an expert's matrices are read
// once per tile of tokens.
#include "common.h"
#include "pta_kernels.h"

// sum over K of w[k] * x_s[k] for one row of W, the lanes of a wave striding over K; every lane gets the sum
template <typename T>
__device__ __forceinline__ float wave_dot(const T* __restrict__ w, const float* __restrict__ x_s, int K, int lane) {
    float acc = 0.f;
    if (sizeof(T) == 4 && (K & 3) == 0 && ((uintptr_t)w & 15) == 0) {
#pragma unroll 4
        for (int k = lane * 4; k < K; k += PTA_WAVE * 4) {
            const float4 f = *reinterpret_cast<const float4*>((const float*)w + k);
            const float4 xv = *reinterpret_cast<const float4*>(x_s + k);
            acc += f.x * xv.x + f.y * xv.y + f.z * xv.z + f.w * xv.w;
        }
    } else if (sizeof(T) == 2 && (K & 7) == 0 && ((uintptr_t)w & 15) == 0) {
#pragma unroll 2
        for (int k = lane * 8; k < K; k += PTA_WAVE * 8) {
            float f[8];
            unpack8(*reinterpret_cast<const uint4*>((const bf16_t*)w + k), f);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc += f[e] * x_s[k + e];
        }
    } else {
        for (int k = lane; k < K; k += PTA_WAVE) acc += Io<T>::ld(w + k) * x_s[k];
    }
    return wave_sum(acc);
}

// the same for NR rows of W `row_ld` apart at once, so that NR loads are on their way for every step over K
template <typename T, int NR>
__device__ __forceinline__ void wave_dots(const T* __restrict__ w, long row_ld, int rows, const float* __restrict__ x_s, int K,
                                          int lane, float (&out)[NR]) {
    float acc[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) acc[r] = 0.f;
    const T* wr[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) wr[r] = w + (long)min(r, rows - 1) * row_ld;  // rows past the last repeat it
    if (sizeof(T) == 2 && (K & 7) == 0 && ((uintptr_t)w & 15) == 0 && (row_ld & 7) == 0) {
#pragma unroll 2
        for (int k = lane * 8; k < K; k += PTA_WAVE * 8) {
            uint4 u[NR];
#pragma unroll
            for (int r = 0; r < NR; ++r) u[r] = *reinterpret_cast<const uint4*>((const bf16_t*)wr[r] + k);
            const float4 x0 = *reinterpret_cast<const float4*>(x_s + k), x1 = *reinterpret_cast<const float4*>(x_s + k + 4);
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                float f[8];
                unpack8(u[r], f);
                acc[r] += f[0] * x0.x + f[1] * x0.y + f[2] * x0.z + f[3] * x0.w + f[4] * x1.x + f[5] * x1.y + f[6] * x1.z + f[7] * x1.w;
            }
        }
    } else {
        for (int k = lane; k < K; k += PTA_WAVE) {
#pragma unroll
            for (int r = 0; r < NR; ++r) acc[r] += Io<T>::ld(wr[r] + k) * x_s[k];
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) out[r] = wave_sum(acc[r]);
}

template <typename T>
__global__ __launch_bounds__(1024) void moe_route_kernel(int* __restrict__ ids, float* __restrict__ wts,
                                                        const T* __restrict__ h, long h_ld, const float* __restrict__ Wr,
                                                        const float* __restrict__ br, int H, int E, int top, int score_kind,
                                                        int normalise, float scale, int groups, int keep,
                                                        const float* __restrict__ extra, float* __restrict__ extra_out,
                                                        int n_extra) {
    extern __shared__ __attribute__((aligned(16))) float sm[];
    float* x_s = sm;       // [H]
    float* s_s = sm + H;   // [E]
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    for (int i = threadIdx.x; i < H; i += blockDim.x) x_s[i] = Io<T>::ld(h + (long)m * h_ld + i);
    __syncthreads();
    for (int e = wave; e < E; e += nw) {
        const float z = wave_dot<float>(Wr + (long)e * H, x_s, H, lane);
        if (lane == 0) s_s[e] = br ? z + br[e] : z;
    }
    for (int e = wave; e < n_extra; e += nw) {
        const float z = wave_dot<float>(extra + (long)e * H, x_s, H, lane);
        if (lane == 0) extra_out[(long)m * n_extra + e] = 1.0f / (1.0f + expf(-z));
    }
    __syncthreads();
    if (wave != 0) return;
    if (score_kind == PTA_ROUTE_SOFTMAX) {
        float mx = -INFINITY;
        for (int e = lane; e < E; e += PTA_WAVE) mx = fmaxf(mx, s_s[e]);
        mx = wave_max(mx);
        float sum = 0.f;
        for (int e = lane; e < E; e += PTA_WAVE) sum += expf(s_s[e] - mx);
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += PTA_WAVE) s_s[e] = expf(s_s[e] - mx) / sum;
    } else {
        for (int e = lane; e < E; e += PTA_WAVE) s_s[e] = 1.0f / (1.0f + expf(-s_s[e]));
    }
    // the largest score `top` times over; of equal scores the expert with the lower index first
    float total = 0.f, mine = 0.f;
    int mine_id = 0;
    unsigned taken = 0;  // bit j: this lane's expert lane + 64 j has been taken (or may not be)
    if (groups > 1 && keep < groups) {
        // lane g holds the score of run g (at most 64 runs); the `keep` best runs stay, the lower index first among equals
        const int size = E / groups;
        float gs = -INFINITY;
        if (lane < groups)
            for (int e = lane * size; e < (lane + 1) * size; ++e) gs = fmaxf(gs, s_s[e]);
        unsigned long long kept = 0ull;
        for (int k = 0; k < keep; ++k) {
            float best = gs;
            int at = lane < groups && !((kept >> lane) & 1ull) ? lane : groups;
            if (at == groups) best = -INFINITY;
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, 64);
                const int oa = __shfl_xor(at, o, 64);
                if (oa < groups && (at == groups || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
            }
            kept |= 1ull << at;
        }
        for (int e = lane, j = 0; e < E; e += PTA_WAVE, ++j)
            if (!((kept >> (e / size)) & 1ull)) taken |= 1u << j;
    }
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = E;
        for (int e = lane, j = 0; e < E; e += PTA_WAVE, ++j) {
            const float v = s_s[e];
            if (!((taken >> j) & 1u) && (v > best || at == E)) { best = v; at = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (oa < E && (at == E || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
        }
        if (lane == k) { mine = best; mine_id = at; }
        total += best;
        if ((at & 63) == lane) taken |= 1u << (at >> 6);
    }
    if (lane < top) {
        ids[(long)m * top + lane] = mine_id;
        wts[(long)m * top + lane] = (normalise ? mine / (total + 1e-20f) : mine) * scale;
    }
}

extern "C" int pta_moe_route(int* ids, float* wts, const void* h, long h_ld, const float* Wr, const float* br, int M, int H, int E, int top,
                             int score_kind, int normalise, float scale, int groups, int keep, const float* extra,
                             float* extra_out, int n_extra, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0 && E > 0 && top > 0, "moe_route: sizes must be positive");
    PTA_REQUIRE(top <= E && top <= 64 && E <= 2048, "moe_route: %d experts per token of %d (at most 64 of at most 2048)", top, E);
    PTA_REQUIRE(ids && wts && h && Wr && h_ld >= H, "moe_route: null pointer or rows too close");
    PTA_REQUIRE(groups >= 1 && groups <= 64 && E % groups == 0 && keep >= 1 && keep <= groups && (long)keep * (E / groups) >= top,
                "moe_route: %d experts in %d groups of which %d are kept do not give %d experts a token", E, groups, keep, top);
    PTA_REQUIRE(n_extra >= 0 && (n_extra == 0 || (extra && extra_out)), "moe_route: further rows need their matrix and a place for the result");
    PTA_REQUIRE(score_kind == PTA_ROUTE_SIGMOID || score_kind == PTA_ROUTE_SOFTMAX, "moe_route: score kind %d is not built", score_kind);
    PTA_REQUIRE((size_t)(H + E) * 4 <= 64 * 1024, "moe_route: %d features and %d experts do not fit the kernel's LDS", H, E);
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_route: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)(H + E) * sizeof(float);
    const dim3 block(E >= 16 ? 1024 : E >= 8 ? 512 : 256);  // a wave an expert where there are that many
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_route_kernel<float>, dim3(M), block, lds, s, ids, wts, (const float*)h, h_ld, Wr, br, H, E, top, score_kind, normalise, scale, groups, keep, extra, extra_out, n_extra);
    else
        hipLaunchKernelGGL(moe_route_kernel<bf16_t>, dim3(M), block, lds, s, ids, wts, (const bf16_t*)h, h_ld, Wr, br, H, E, top, score_kind, normalise, scale, groups, keep, extra, extra_out, n_extra);
    return pta_check_launch("moe_route");
}

#define MOE_ROWS 16  // rows of an expert's matrix per workgroup of four waves

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(T* __restrict__ act_out, const T* __restrict__ h, long h_ld,
                                                     const T* __restrict__ gate_up, const int* __restrict__ ids, int H,
                                                     int F, int top, int act, PtaGate gate, int gated) {
    extern __shared__ __attribute__((aligned(16))) float x_s[];  // [H]
    const int pair = blockIdx.x, m = pair / top, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int e = ids[pair];
    for (int i = threadIdx.x; i < H; i += blockDim.x) x_s[i] = Io<T>::ld(h + (long)m * h_ld + i);
    __syncthreads();
    const T* G = gate_up + (long)e * (gated ? 2 : 1) * F * H;
    const T* U = G + (long)F * H;
    // a wave takes four neighbouring rows of the gate and of the up matrix: eight loads on their way at once
    const int f0 = blockIdx.y * MOE_ROWS + wave * 4, rows = min(4, F - f0);
    if (rows <= 0) return;
    float g[4], u[4];
    wave_dots<T, 4>(G + (long)f0 * H, H, rows, x_s, H, lane, g);
    if (!gated) {  // an expert without a gate: act of its one product
        if (lane < rows) {
            float gv = g[0];
#pragma unroll
            for (int r = 1; r < 4; ++r)
                if (lane == r) gv = g[r];
            Io<T>::st(act_out + (long)pair * F + f0 + lane, apply_act(Io<T>::round(gv), act));
        }
        return;
    }
    wave_dots<T, 4>(U + (long)f0 * H, H, rows, x_s, H, lane, u);
    // (each product rounded to the compute type first, as a product on its own would leave it)
    if (lane < rows) {
        float gv = g[0], uv = u[0];
#pragma unroll
        for (int r = 1; r < 4; ++r)
            if (lane == r) { gv = g[r]; uv = u[r]; }
        Io<T>::st(act_out + (long)pair * F + f0 + lane, gate_value(Io<T>::round(gv), Io<T>::round(uv), act, gate));
    }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(T* __restrict__ out, const T* __restrict__ act_in,
                                                       const T* __restrict__ down, const int* __restrict__ ids,
                                                       const float* __restrict__ wts, int H, int F, int top,
                                                       const T* __restrict__ extra, const float* __restrict__ extra_gate,
                                                       int gate_ld) {
    extern __shared__ __attribute__((aligned(16))) float a_s[];  // [top][F]
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < top * F; i += blockDim.x) a_s[i] = Io<T>::ld(act_in + (long)m * top * F + i);
    __syncthreads();
    const int n0 = blockIdx.y * MOE_ROWS + wave * 4, rows = min(4, H - n0);
    if (rows <= 0) return;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int k = 0; k < top; ++k) {
        float d[4];
        wave_dots<T, 4>(down + ((long)ids[(long)m * top + k] * H + n0) * F, F, rows, a_s + k * F, F, lane, d);
        const float wk = wts[(long)m * top + k];
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += wk * Io<T>::round(d[r]);
    }
    if (lane < rows) {
        float v = acc[0];
#pragma unroll
        for (int r = 1; r < 4; ++r)
            if (lane == r) v = acc[r];
        if (extra) v += extra_gate[(long)m * gate_ld] * Io<T>::ld(extra + (long)m * H + n0 + lane);
        Io<T>::st(out + (long)m * H + n0 + lane, v);
    }
}

// act_out [M * top, F]; h [M, H] rows h_ld apart; gate_up [E, 2F, H] (gated) or [E, F, H]; ids [M, top]
extern "C" int pta_moe_up(void* act_out, const void* h, long h_ld, const void* gate_up, const int* ids, int M, int H, int F,
                          int top, int act, const PtaGate* gate_how, int gated, int dtype, void* stream) {
    const PtaGate gate = gate_how ? *gate_how : PtaGate{PTA_GLU_SILU, 1.f, 0.f};
    PTA_REQUIRE(gate.kind == PTA_GLU_SILU || gate.kind == PTA_GLU_CLAMPED, "moe_up: a gate of kind %d is not built", gate.kind);
    PTA_REQUIRE(M > 0 && H > 0 && F > 0 && top > 0 && act_out && h && gate_up && ids && h_ld >= H, "moe_up: sizes must be positive and pointers given");
    PTA_REQUIRE(pta_act_known(act), "moe_up: unknown activation %d", act);
    PTA_REQUIRE((size_t)H * 4 <= 64 * 1024 && (F + MOE_ROWS - 1) / MOE_ROWS <= 65535, "moe_up: sizes beyond one launch");
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_up: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid((unsigned)((long)M * top), (F + MOE_ROWS - 1) / MOE_ROWS);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_up_kernel<float>, grid, dim3(256), (size_t)H * 4, s, (float*)act_out, (const float*)h, h_ld, (const float*)gate_up, ids, H, F, top, act, gate, gated);
    else
        hipLaunchKernelGGL(moe_up_kernel<bf16_t>, grid, dim3(256), (size_t)H * 4, s, (bf16_t*)act_out, (const bf16_t*)h, h_ld, (const bf16_t*)gate_up, ids, H, F, top, act, gate, gated);
    return pta_check_launch("moe_up");
}

// out [M, H]; act_in [M * top, F]; down [E, H, F]
// extra [M, H] (compute type) and extra_gate (32-bit, one number a token, gate_ld apart), both or neither: out += gate * extra
extern "C" int pta_moe_down(void* out, const void* act_in, const void* down, const int* ids, const float* wts, int M, int H,
                            int F, int top, const void* extra, const float* extra_gate, int gate_ld, int dtype, void* stream) {
    PTA_REQUIRE((extra != nullptr) == (extra_gate != nullptr), "moe_down: a further term and its gate come together");
    PTA_REQUIRE(M > 0 && H > 0 && F > 0 && top > 0 && out && act_in && down && ids && wts, "moe_down: sizes must be positive and pointers given");
    PTA_REQUIRE((size_t)top * F * 4 <= 160 * 1024 && (H + MOE_ROWS - 1) / MOE_ROWS <= 65535,
                "moe_down: %d experts of %d rows a token are more than the kernel's LDS holds", top, F);
    PTA_REQUIRE(dtype == PTA_F32 || dtype == PTA_BF16, "moe_down: unknown dtype %d", dtype);
    hipStream_t s = (hipStream_t)stream;
    if ((size_t)top * F * 4 > 64 * 1024) {  // more than a launch may ask for unless the kernel has been told
        const void* kern = dtype == PTA_F32 ? reinterpret_cast<const void*>(moe_down_kernel<float>)
                                            : reinterpret_cast<const void*>(moe_down_kernel<bf16_t>);
        (void)hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)((size_t)top * F * 4));
    }
    const dim3 grid(M, (H + MOE_ROWS - 1) / MOE_ROWS);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(moe_down_kernel<float>, grid, dim3(256), (size_t)top * F * 4, s, (float*)out, (const float*)act_in, (const float*)down, ids, wts, H, F, top, (const float*)extra, extra_gate, gate_ld);
    else
        hipLaunchKernelGGL(moe_down_kernel<bf16_t>, grid, dim3(256), (size_t)top * F * 4, s, (bf16_t*)out, (const bf16_t*)act_in, (const bf16_t*)down, ids, wts, H, F, top, (const bf16_t*)extra, extra_gate, gate_ld);
    return pta_check_launch("moe_down");
}

// ---- steps of many tokens: tiles of one expert's tokens on the matrix cores --------------------------------------------
// pta_moe_sort lays the (token, expert) pairs out by expert: every expert's pairs take a run of slots that starts at a
// multiple of MOE_TILE, the slots between an expert's last pair and the next multiple hold -1.  tile_expert[t] is the
// expert of slots t * MOE_TILE .. + MOE_TILE - 1 (-1: no such tile), slot_of_pair[p] where pair p went.  One workgroup;
// the order of an expert's pairs among themselves is whatever the atomics give, and no result depends on it (a row's
// products are the same sums wherever the row lies).
#define MOE_TILE 64

__global__ __launch_bounds__(1024) void moe_sort_kernel(int* __restrict__ sorted_pair, int* __restrict__ slot_of_pair,
                                                        int* __restrict__ tile_expert, const int* __restrict__ ids, int pairs,
                                                        int E, int slots, int tiles) {
    extern __shared__ int sm_i[];
    int* count = sm_i;          // [E]
    int* start = sm_i + E;      // [E + 1], in slots
    int* cursor = start + E + 1;  // [E]
    for (int e = threadIdx.x; e < E; e += blockDim.x) { count[e] = 0; cursor[e] = 0; }
    for (int i = threadIdx.x; i < slots; i += blockDim.x) sorted_pair[i] = -1;
    for (int t = threadIdx.x; t < tiles; t += blockDim.x) tile_expert[t] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) atomicAdd(&count[ids[p]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < E; ++e) {
            start[e] = at;
            at += (count[e] + MOE_TILE - 1) / MOE_TILE * MOE_TILE;
        }
        start[E] = at;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += blockDim.x)
        for (int t = start[e] / MOE_TILE; t < start[e + 1] / MOE_TILE; ++t) tile_expert[t] = e;
    for (int p = threadIdx.x; p < pairs; p += blockDim.x) {
        const int e = ids[p];
        const int slot = start[e] + atomicAdd(&cursor[e], 1);
        sorted_pair[slot] = p;
        slot_of_pair[p] = slot;
    }
}

typedef __bf16 moe_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float moe_f32x4_t __attribute__((ext_vector_type(4)));
union MoeFrag { uint4 u; moe_bf16x8_t v; };

__device__ __forceinline__ uint32_t moe_pack2(float lo, float hi) {
    return (uint32_t)f32_to_bf16_bits(lo) | ((uint32_t)f32_to_bf16_bits(hi) << 16);
}

// The products of a tile: C^T[row of W][slot] += W rows . B rows over K, for NA groups of sixteen W rows a wave and the
// tile's four groups of sixteen slots.  W rows are the matrix cores' A operand, sixteen bytes of a row per lane,
// straight from memory and asked for one step of 32 ahead; the tile's B rows (64 slots x 64 elements of K a stage) go
// through LDS, which the four waves of the workgroup share, two stages in turn with one barrier a stage.
#define MOE_STAGE 64
#define MOE_XROW 72  // elements between two rows of a stage in LDS: 144 bytes, so that sixteen rows spread over the banks

template <int NA>
__device__ __forceinline__ void moe_tile_products(moe_f32x4_t (&acc)[NA][4], const bf16_t* const (&arow)[NA],
                                                  const bf16_t* brow, int K, bf16_t* lds) {
    const int tid = threadIdx.x, lane = tid & 63, c = lane & 15, gq = lane >> 4;
    const int st_at = (tid >> 2) * MOE_XROW + (tid & 3) * 8;  // where this thread puts its two pieces of a stage
#pragma unroll
    for (int a = 0; a < NA; ++a)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[a][tt] = moe_f32x4_t{0.f, 0.f, 0.f, 0.f};
    uint4 g0 = *reinterpret_cast<const uint4*>(brow), g1 = *reinterpret_cast<const uint4*>(brow + 32);
    MoeFrag wn[2][NA];  // the W rows' pieces of the stage to come: asked for a stage (two steps of 32) ahead
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int a = 0; a < NA; ++a) wn[ks][a].u = *reinterpret_cast<const uint4*>(arow[a] + ks * 32);
    *reinterpret_cast<uint4*>(lds + st_at) = g0;
    *reinterpret_cast<uint4*>(lds + st_at + 32) = g1;
    __syncthreads();
    const int stages = K / MOE_STAGE;
    for (int s = 0; s < stages; ++s) {
        const bf16_t* cur = lds + (s & 1) * (MOE_TILE * MOE_XROW);
        const bool more = s + 1 < stages;
        MoeFrag wc[2][NA];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int a = 0; a < NA; ++a) wc[ks][a] = wn[ks][a];
        if (more) {
            g0 = *reinterpret_cast<const uint4*>(brow + (s + 1) * MOE_STAGE);
            g1 = *reinterpret_cast<const uint4*>(brow + (s + 1) * MOE_STAGE + 32);
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int a = 0; a < NA; ++a)
                    wn[ks][a].u = *reinterpret_cast<const uint4*>(arow[a] + (s + 1) * MOE_STAGE + ks * 32);
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            MoeFrag xb[4];
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
                xb[tt].u = *reinterpret_cast<const uint4*>(cur + (tt * 16 + c) * MOE_XROW + ks * 32 + gq * 8);
#pragma unroll
            for (int a = 0; a < NA; ++a)
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
                    acc[a][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wc[ks][a].v, xb[tt].v, acc[a][tt], 0, 0, 0);
        }
        if (more) {
            bf16_t* nxt = lds + ((s + 1) & 1) * (MOE_TILE * MOE_XROW);
            *reinterpret_cast<uint4*>(nxt + st_at) = g0;
            *reinterpret_cast<uint4*>(nxt + st_at + 32) = g1;
        }
        __syncthreads();
    }
}

// Which (tile, block of W rows) a workgroup takes.  Workgroups go to the chip's eight dies in turn, each die with a cache
// of its own; the tiles of one expert against one block of its rows read the same W, so they are handed to one die, one
// after the other: workgroup L takes the L / 8-th item of die L % 8's share of the list ordered by (block, tile).
__device__ __forceinline__ bool moe_item(int tiles, int blocks, int* tile, int* block) {
    const int total = tiles * blocks, per = (total + 7) / 8;
    const int L = blockIdx.x, item = (L % 8) * per + L / 8;
    if (L / 8 >= per || item >= total) return false;
    *block = item / tiles;
    *tile = item - *block * tiles;
    return true;
}

// four values of one slot's row, rows r .. r + 3 of `limit`, as bfloat16
__device__ __forceinline__ void moe_store4(bf16_t* dst, int r, int limit, float y0, float y1, float y2, float y3) {
    if (r + 3 < limit) {
        uint2 w2;
        w2.x = moe_pack2(y0, y1);
        w2.y = moe_pack2(y2, y3);
        *reinterpret_cast<uint2*>(dst) = w2;
    } else {
        const float y[4] = {y0, y1, y2, y3};
        for (int j = 0; j < 4; ++j)
            if (r + j < limit) dst[j] = f32_to_bf16_bits(y[j]);
    }
}

// act_sorted[slot, f] = act(G_e x) * (U_e x) for the slot's pair (token, e).  A workgroup of four waves owns a tile of
// MOE_TILE slots and 128 rows f of its expert; a wave 32 rows of the gate and the same 32 of the up matrix.
__global__ __launch_bounds__(256) void moe_grouped_up_kernel(bf16_t* __restrict__ act_sorted, const bf16_t* __restrict__ x,
                                                             long x_ld, const bf16_t* __restrict__ gate_up,
                                                             const int* __restrict__ sorted_pair,
                                                             const int* __restrict__ tile_expert, int H, int F, int top,
                                                             int act, PtaGate gate, int tiles) {
    __shared__ __attribute__((aligned(16))) bf16_t lds[2 * MOE_TILE * MOE_XROW];
    int tile, fb;
    if (!moe_item(tiles, (F + 127) / 128, &tile, &fb)) return;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, gq = lane >> 4;
    const int f0 = fb * 128 + wave * 32;
    const bf16_t* W = gate_up + (long)e * 2 * F * H + gq * 8;
    const bf16_t* arow[4];
#pragma unroll
    for (int a = 0; a < 4; ++a)  // gate rows f0 .. f0 + 31, then the same rows of the up matrix
        arow[a] = W + ((long)(a >> 1) * F + min(f0 + (a & 1) * 16 + c, F - 1)) * H;
    const int pair = sorted_pair[tile * MOE_TILE + (tid >> 2)];
    const bf16_t* brow = x + (long)(pair < 0 ? 0 : pair / top) * x_ld + (tid & 3) * 8;
    moe_f32x4_t acc[4][4];
    moe_tile_products<4>(acc, arow, brow, H, lds);
    if (f0 >= F) return;
    // acc[a][tt][j] is row f0 + (a & 1) * 16 + 4 gq + j of the slot in column c of group tt
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const long slot = (long)tile * MOE_TILE + tt * 16 + c;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float y[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
                y[j] = gate_value(round_to_bf16(acc[half][tt][j]), round_to_bf16(acc[2 + half][tt][j]), act, gate);
            const int f = f0 + half * 16 + 4 * gq;
            moe_store4(act_sorted + slot * F + f, f, F, y[0], y[1], y[2], y[3]);
        }
    }
}

// The same for experts without a gate: act_sorted[slot, f] = act(U_e x).  A wave owns four groups of sixteen rows f of the
// expert's one input matrix, a workgroup 256 rows.
__global__ __launch_bounds__(256) void moe_grouped_up_plain_kernel(bf16_t* __restrict__ act_sorted, const bf16_t* __restrict__ x,
                                                                   long x_ld, const bf16_t* __restrict__ up,
                                                                   const int* __restrict__ sorted_pair,
                                                                   const int* __restrict__ tile_expert, int H, int F, int top,
                                                                   int act, int tiles) {
    __shared__ __attribute__((aligned(16))) bf16_t lds[2 * MOE_TILE * MOE_XROW];
    int tile, fb;
    if (!moe_item(tiles, (F + 255) / 256, &tile, &fb)) return;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, gq = lane >> 4;
    const int f0 = fb * 256 + wave * 64;
    const bf16_t* arow[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) arow[a] = up + ((long)e * F + min(f0 + a * 16 + c, F - 1)) * H + gq * 8;
    const int pair = sorted_pair[tile * MOE_TILE + (tid >> 2)];
    const bf16_t* brow = x + (long)(pair < 0 ? 0 : pair / top) * x_ld + (tid & 3) * 8;
    moe_f32x4_t acc[4][4];
    moe_tile_products<4>(acc, arow, brow, H, lds);
    if (f0 >= F) return;
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const long slot = (long)tile * MOE_TILE + tt * 16 + c;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            float y[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) y[j] = apply_act(round_to_bf16(acc[a][tt][j]), act);
            const int f = f0 + a * 16 + 4 * gq;
            moe_store4(act_sorted + slot * F + f, f, F, y[0], y[1], y[2], y[3]);
        }
    }
}

// y_sorted[slot, n] = D_e act_sorted[slot]: a wave owns four groups of sixteen rows n of the expert's down matrix, a
// workgroup 256 rows, against the tile's 64 slots
__global__ __launch_bounds__(256) void moe_grouped_down_kernel(bf16_t* __restrict__ y_sorted, const bf16_t* __restrict__ act_sorted,
                                                               const bf16_t* __restrict__ down,
                                                               const int* __restrict__ tile_expert, int H, int F, int tiles) {
    __shared__ __attribute__((aligned(16))) bf16_t lds[2 * MOE_TILE * MOE_XROW];
    int tile, nb;
    if (!moe_item(tiles, (H + 255) / 256, &tile, &nb)) return;
    const int e = tile_expert[tile];
    if (e < 0) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, gq = lane >> 4;
    const int n0 = nb * 256 + wave * 64;
    const bf16_t* arow[4];
#pragma unroll
    for (int a = 0; a < 4; ++a) arow[a] = down + ((long)e * H + min(n0 + a * 16 + c, H - 1)) * F + gq * 8;
    const bf16_t* brow = act_sorted + ((long)tile * MOE_TILE + (tid >> 2)) * F + (tid & 3) * 8;
    moe_f32x4_t acc[4][4];
    moe_tile_products<4>(acc, arow, brow, F, lds);
    if (n0 >= H) return;
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) {
        const long slot = (long)tile * MOE_TILE + tt * 16 + c;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int n = n0 + a * 16 + 4 * gq;
            moe_store4(y_sorted + slot * H + n, n, H, acc[a][tt][0], acc[a][tt][1], acc[a][tt][2], acc[a][tt][3]);
        }
    }
}

// out[m, n] = sum_k wts[m, k] * y_sorted[slot_of_pair[m * top + k], n], in the order the experts were taken
__global__ void moe_combine_kernel(bf16_t* __restrict__ out, const bf16_t* __restrict__ y_sorted,
                                   const int* __restrict__ slot_of_pair, const float* __restrict__ wts, int H, int top,
                                   const bf16_t* __restrict__ extra, const float* __restrict__ extra_gate, int gate_ld) {
    const int m = blockIdx.x;
    for (int n = threadIdx.x; n < H; n += blockDim.x) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k)
            acc += wts[(long)m * top + k] * bf16_bits_to_f32(y_sorted[(long)slot_of_pair[(long)m * top + k] * H + n]);
        if (extra) acc += extra_gate[(long)m * gate_ld] * bf16_bits_to_f32(extra[(long)m * H + n]);
        out[(long)m * H + n] = f32_to_bf16_bits(acc);
    }
}

extern "C" int pta_moe_grouped_slots(int pairs, int E) { return (pairs + E * (MOE_TILE - 1) + MOE_TILE - 1) / MOE_TILE * MOE_TILE; }

// bfloat16 only; H and F multiples of 64.  sorted_pair [slots], slot_of_pair [M * top], tile_expert [slots / 64],
// act_sorted [slots, F], y_sorted [slots, H] are the caller's scratch (slots = pta_moe_grouped_slots(M * top, E)).
extern "C" int pta_moe_grouped(void* out, const void* x, long x_ld, const void* gate_up, const void* down, const int* ids,
                               const float* wts, int* sorted_pair, int* slot_of_pair, int* tile_expert, void* act_sorted,
                               void* y_sorted, int M, int H, int F, int E, int top, int act, const PtaGate* gate_how,
                               int gated, const void* extra, const float* extra_gate, int gate_ld, void* stream) {
    PTA_REQUIRE((extra != nullptr) == (extra_gate != nullptr), "moe_grouped: a further term and its gate come together");
    const PtaGate gate = gate_how ? *gate_how : PtaGate{PTA_GLU_SILU, 1.f, 0.f};
    PTA_REQUIRE(gate.kind == PTA_GLU_SILU || gate.kind == PTA_GLU_CLAMPED, "moe_grouped: a gate of kind %d is not built", gate.kind);
    PTA_REQUIRE(M > 0 && H > 0 && F > 0 && E > 0 && top > 0, "moe_grouped: sizes must be positive");
    PTA_REQUIRE(H % 64 == 0 && F % 64 == 0 && x_ld % 8 == 0, "moe_grouped: features (%d) and expert size (%d) must be multiples of 64", H, F);
    PTA_REQUIRE(out && x && gate_up && down && ids && wts && sorted_pair && slot_of_pair && tile_expert && act_sorted && y_sorted,
                "moe_grouped: null pointer");
    PTA_REQUIRE((((uintptr_t)x | (uintptr_t)gate_up | (uintptr_t)down | (uintptr_t)act_sorted | (uintptr_t)y_sorted) % 16) == 0,
                "moe_grouped: matrices must be aligned to sixteen bytes");
    PTA_REQUIRE(pta_act_known(act), "moe_grouped: unknown activation %d", act);
    PTA_REQUIRE((size_t)(3 * E + 1) * 4 <= 64 * 1024, "moe_grouped: %d experts are more than the sort holds", E);
    const long pairs = (long)M * top;
    const int slots = pta_moe_grouped_slots((int)pairs, E), tiles = slots / MOE_TILE;
    PTA_REQUIRE(pairs < (1L << 30) && tiles <= 2147483647 / 64, "moe_grouped: too many pairs");
    hipStream_t s = (hipStream_t)stream;
    hipLaunchKernelGGL(moe_sort_kernel, dim3(1), dim3(1024), (size_t)(3 * E + 1) * 4, s, sorted_pair, slot_of_pair, tile_expert,
                       ids, (int)pairs, E, slots, tiles);
    auto grid_for = [&](int blocks) { return dim3((unsigned)(((long)tiles * blocks + 7) / 8 * 8)); };
    if (gated)
        hipLaunchKernelGGL(moe_grouped_up_kernel, grid_for((F + 127) / 128), dim3(256), 0, s, (bf16_t*)act_sorted, (const bf16_t*)x,
                           x_ld, (const bf16_t*)gate_up, sorted_pair, tile_expert, H, F, top, act, gate, tiles);
    else
        hipLaunchKernelGGL(moe_grouped_up_plain_kernel, grid_for((F + 255) / 256), dim3(256), 0, s, (bf16_t*)act_sorted,
                           (const bf16_t*)x, x_ld, (const bf16_t*)gate_up, sorted_pair, tile_expert, H, F, top, act, tiles);
    hipLaunchKernelGGL(moe_grouped_down_kernel, grid_for((H + 255) / 256), dim3(256), 0, s, (bf16_t*)y_sorted,
                       (const bf16_t*)act_sorted, (const bf16_t*)down, tile_expert, H, F, tiles);
    hipLaunchKernelGGL(moe_combine_kernel, dim3(M), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)y_sorted, slot_of_pair, wts, H, top,
                       (const bf16_t*)extra, extra_gate, gate_ld);
    return pta_check_launch("moe_grouped");
}
