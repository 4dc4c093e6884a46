// A feed-forward made of many small gated ones ("experts"), of which a router chooses a few per token.
//
//   vt_moe_route:    logits z = W_r x in float32 (W_r is kept in float32), scores sigmoid(z) or softmax(z), the `top`
//                    largest per token (the lower index among equals), optionally divided by their sum.  A wave per token.
//   vt_moe_gate_up:  for every (token, choice): act = f(W_gate,e xe) * (W_up,e xe), where xe is the token's input times
//                    in_scale (the choice's score where the score multiplies the expert's input, else 1), rounded to the
//                    runtime's type as an expert's input is; f(g) = g sigmoid(alpha g (1 + cubic g^2)).
//   vt_moe_down:     out[t] = sum over the token's choices, in their order, of out_scale * W_down,e act.
// These two read an expert's matrices once per token that chose it: the arrangement for few tokens, where every chosen
// expert's matrices have to be read anyway.  (Many tokens go through vt_moe_sort and the grouped products below.)
// Every sum is taken in an order that depends on the sizes alone, so a token's result does not depend on its batch.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

template <typename TI>
__global__ __launch_bounds__(64) void moe_route_kernel(const TI* __restrict__ x, const float* __restrict__ wr,
                                                       int* __restrict__ ids, float* __restrict__ wts, int E, int W, int top,
                                                       int softmax, int renorm) {
    extern __shared__ float sc[];       // E scores
    const int t = blockIdx.x, lane = threadIdx.x;
    const TI* xt = x + (size_t)t * W;
    for (int e = 0; e < E; ++e) {
        const float* row = wr + (size_t)e * W;
        float acc = 0.f;
        for (int j = lane; j < W; j += 64) acc = fmaf(row[j], load_f32<TI>(xt, j), acc);
        acc = wave_sum(acc);
        if (lane == 0) sc[e] = acc;
    }
    wave_lds_order();
    if (softmax) {
        float m = -INFINITY;
        for (int e = lane; e < E; e += 64) m = fmaxf(m, sc[e]);
        m = wave_max(m);
        float s = 0.f;
        for (int e = lane; e < E; e += 64) s += expf(sc[e] - m);
        s = wave_sum(s);
        wave_lds_order();
        for (int e = lane; e < E; e += 64) sc[e] = expf(sc[e] - m) / s;
    } else {
        for (int e = lane; e < E; e += 64) sc[e] = 1.0f / (1.0f + expf(-sc[e]));
    }
    wave_lds_order();
    float total = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float v = sc[e];
            if (v > best) { best = v; at = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (at == 0x7fffffff) at = k < E ? k : 0;     // scores that are no numbers: some expert all the same
        total += best;
        if (lane == 0) {
            ids[(size_t)t * top + k] = at;
            wts[(size_t)t * top + k] = best;
            sc[at] = -INFINITY;
        }
        wave_lds_order();
    }
    if (renorm && lane == 0)
        for (int k = 0; k < top; ++k) wts[(size_t)t * top + k] /= total;
}

extern "C" int vt_moe_route(const void* x, int dtype, const float* wr, int* ids, float* wts, int n, int E, int W, int top,
                            int softmax, int renorm, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && E > 0 && W > 0 && top > 0 && top <= E, "vt_moe_route: bad sizes n=%d E=%d W=%d top=%d", n, E, W, top);
    VT_REQUIRE(E <= 8192, "vt_moe_route: %d experts (up to 8192)", E);
    if (n == 0) return 0;
    const size_t lds = (size_t)E * sizeof(float);
    if (dtype == VT_F32) moe_route_kernel<float><<<n, 64, lds, stream>>>((const float*)x, wr, ids, wts, E, W, top, softmax, renorm);
    else if (dtype == VT_BF16) moe_route_kernel<bf16_t><<<n, 64, lds, stream>>>((const bf16_t*)x, wr, ids, wts, E, W, top, softmax, renorm);
    else return vt_fail("vt_moe_route: unknown dtype %d", dtype);
    VT_CHECK_LAUNCH("vt_moe_route");
    return 0;
}

// ---------------------------------------------------------------------------
// a wave's dot product of a matrix row with a vector in LDS: lanes take eight elements at a time where the row allows
// 16-byte loads, one at a time otherwise; the lanes' shares are added by the butterfly of wave_sum
template <typename TW>
__device__ __forceinline__ float wave_dot(const TW* __restrict__ row, const float* __restrict__ v, int K, int lane) {
    float acc = 0.f;
    if constexpr (sizeof(TW) == 2) {
        if (K % 8 == 0 && !((uintptr_t)row & 15)) {
            typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));
            for (int j = lane * 8; j < K; j += 512) {
                const u32x4_t w = *(const u32x4_t*)(row + j);
                acc = fmaf(lowp_lo(w.x), v[j], acc);     acc = fmaf(lowp_hi(w.x), v[j + 1], acc);
                acc = fmaf(lowp_lo(w.y), v[j + 2], acc); acc = fmaf(lowp_hi(w.y), v[j + 3], acc);
                acc = fmaf(lowp_lo(w.z), v[j + 4], acc); acc = fmaf(lowp_hi(w.z), v[j + 5], acc);
                acc = fmaf(lowp_lo(w.w), v[j + 6], acc); acc = fmaf(lowp_hi(w.w), v[j + 7], acc);
            }
            return wave_sum(acc);
        }
    }
    for (int j = lane; j < K; j += 64) acc = fmaf(load_f32<TW>(row, j), v[j], acc);
    return wave_sum(acc);
}

#define MOE_OUTS_PER_WAVE 4
#define MOE_OUTS_PER_BLOCK (4 * MOE_OUTS_PER_WAVE)

// w_gu: [E][2 * F][W] (an expert's gate rows, then its up rows); act: [pairs][F]
template <typename TI, typename TW>
__global__ __launch_bounds__(256) void moe_gate_up_kernel(const TI* __restrict__ x, const TW* __restrict__ w_gu,
                                                          const int* __restrict__ ids, const float* __restrict__ wts,
                                                          TI* __restrict__ act, int W, int F, int top, int scale_input,
                                                          float alpha, float cubic) {
    extern __shared__ float xs[];       // W
    const int p = blockIdx.x;
    const int t = p / top;
    const int e = ids[p];
    const float s = scale_input ? wts[p] : 1.0f;
    for (int j = threadIdx.x; j < W; j += 256) {
        float v = load_f32<TI>(x, (size_t)t * W + j) * s;
        if constexpr (sizeof(TI) == 2) v = bf16_to_f32(f32_to_bf16(v));
        xs[j] = v;
    }
    __syncthreads();
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const TW* we = w_gu + (size_t)e * 2 * F * W;
#pragma unroll
    for (int i = 0; i < MOE_OUTS_PER_WAVE; ++i) {
        const int f = blockIdx.y * MOE_OUTS_PER_BLOCK + wave * MOE_OUTS_PER_WAVE + i;
        if (f >= F) break;
        const float g = wave_dot<TW>(we + (size_t)f * W, xs, W, lane);
        const float u = wave_dot<TW>(we + (size_t)(F + f) * W, xs, W, lane);
        if (lane == 0) {
            const float z = cubic != 0.f ? alpha * g * fmaf(cubic * g, g, 1.f) : alpha * g;
            store_f32<TI>(act, (size_t)p * F + f, g / (1.0f + expf(-z)) * u);
        }
    }
}

// w_down: [E][W][F]; out [n][W] float32
template <typename TI, typename TW>
__global__ __launch_bounds__(256) void moe_down_kernel(const TI* __restrict__ act, const TW* __restrict__ w_down,
                                                       const int* __restrict__ ids, const float* __restrict__ wts,
                                                       float* __restrict__ out, int W, int F, int top, int scale_output) {
    extern __shared__ float as[];       // F
    const int t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    float acc[MOE_OUTS_PER_WAVE];
#pragma unroll
    for (int i = 0; i < MOE_OUTS_PER_WAVE; ++i) acc[i] = 0.f;
    for (int k = 0; k < top; ++k) {
        const int p = t * top + k;
        const int e = ids[p];
        const float s = scale_output ? wts[p] : 1.0f;
        __syncthreads();
        for (int f = threadIdx.x; f < F; f += 256) as[f] = load_f32<TI>(act, (size_t)p * F + f);
        __syncthreads();
        const TW* we = w_down + (size_t)e * W * F;
#pragma unroll
        for (int i = 0; i < MOE_OUTS_PER_WAVE; ++i) {
            const int j = blockIdx.y * MOE_OUTS_PER_BLOCK + wave * MOE_OUTS_PER_WAVE + i;
            if (j < W) acc[i] = fmaf(s, wave_dot<TW>(we + (size_t)j * F, as, F, lane), acc[i]);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int i = 0; i < MOE_OUTS_PER_WAVE; ++i) {
            const int j = blockIdx.y * MOE_OUTS_PER_BLOCK + wave * MOE_OUTS_PER_WAVE + i;
            if (j < W) out[(size_t)t * W + j] = acc[i];
        }
    }
}

extern "C" int vt_moe_gate_up(const void* x, int dtype, const void* w_gu, int w_dtype, const int* ids, const float* wts,
                              void* act, int n, int E, int W, int F, int top, int scale_input, float alpha, float cubic,
                              hipStream_t stream) {
    VT_REQUIRE(n >= 0 && E > 0 && W > 0 && F > 0 && top > 0, "vt_moe_gate_up: bad sizes");
    VT_REQUIRE(W <= 16384 && (F + MOE_OUTS_PER_BLOCK - 1) / MOE_OUTS_PER_BLOCK <= 65535, "vt_moe_gate_up: width %d or experts' size %d is too large", W, F);
    VT_REQUIRE(alpha > 0.f, "vt_moe_gate_up: bad gate");
    if (n == 0) return 0;
    const dim3 grid(n * top, (F + MOE_OUTS_PER_BLOCK - 1) / MOE_OUTS_PER_BLOCK);
    const size_t lds = (size_t)W * sizeof(float);
    if (dtype == VT_F32 && w_dtype == VT_F32)
        moe_gate_up_kernel<float, float><<<grid, 256, lds, stream>>>((const float*)x, (const float*)w_gu, ids, wts, (float*)act, W, F, top, scale_input, alpha, cubic);
    else if (dtype == VT_BF16 && w_dtype == VT_BF16)
        moe_gate_up_kernel<bf16_t, bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)x, (const bf16_t*)w_gu, ids, wts, (bf16_t*)act, W, F, top, scale_input, alpha, cubic);
    else return vt_fail("vt_moe_gate_up: dtypes %d / %d are not handled", dtype, w_dtype);
    VT_CHECK_LAUNCH("vt_moe_gate_up");
    return 0;
}

extern "C" int vt_moe_down(const void* act, int dtype, const void* w_down, int w_dtype, const int* ids, const float* wts,
                           float* out, int n, int E, int W, int F, int top, int scale_output, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && E > 0 && W > 0 && F > 0 && top > 0, "vt_moe_down: bad sizes");
    VT_REQUIRE(F <= 16384 && (W + MOE_OUTS_PER_BLOCK - 1) / MOE_OUTS_PER_BLOCK <= 65535, "vt_moe_down: width %d or experts' size %d is too large", W, F);
    if (n == 0) return 0;
    const dim3 grid(n, (W + MOE_OUTS_PER_BLOCK - 1) / MOE_OUTS_PER_BLOCK);
    const size_t lds = (size_t)F * sizeof(float);
    if (dtype == VT_F32 && w_dtype == VT_F32)
        moe_down_kernel<float, float><<<grid, 256, lds, stream>>>((const float*)act, (const float*)w_down, ids, wts, out, W, F, top, scale_output);
    else if (dtype == VT_BF16 && w_dtype == VT_BF16)
        moe_down_kernel<bf16_t, bf16_t><<<grid, 256, lds, stream>>>((const bf16_t*)act, (const bf16_t*)w_down, ids, wts, out, W, F, top, scale_output);
    else return vt_fail("vt_moe_down: dtypes %d / %d are not handled", dtype, w_dtype);
    VT_CHECK_LAUNCH("vt_moe_down");
    return 0;
}
