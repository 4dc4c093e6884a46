// Several residual streams per token ("hyper-connections"), and the blend of a sublayer's input with the previous
// token's ("token shift").  The streams are float32, laid out [token][stream][width].
//
//   vt_streams_fill:   every stream of a token starts as the same vector (the embedding's output).
//   vt_streams_read:   u = sum_s w_in[s] x_s, then RMSNorm: out = (gain * u) / sqrt(mean(u^2) + eps).  With `rows`, only
//                      those tokens (the rows whose logits are wanted).  The sum runs over s = 0, 1, .. in that order and
//                      the row's sum of squares in an order that depends on the block's size alone.
//   vt_streams_write:  x_t <- sum_s mix[s][t] x_s + w_out[t] * y * sigmoid(gate), all streams at once from the old
//                      ones; `gate` (the logits of a sigmoid gate on the sublayer's result) may be absent.
//   vt_token_shift:    out[t] = h[t] + (h[t - 1] - h[t]) * mu, where the token before a step's first token of a request
//                      comes from the request's state (zeros at the start of a sequence); the state then takes the
//                      request's last h of this step.  The thread that reads a state element is the one that writes it.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

#define STREAMS_MAX 8

__global__ __launch_bounds__(256) void streams_fill_kernel(const float* __restrict__ h, float* __restrict__ x, int S, int W,
                                                           long long total) {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const long long t = i / W;
        const int j = (int)(i - t * W);
        const float v = h[i];
        for (int s = 0; s < S; ++s) x[((size_t)t * S + s) * W + j] = v;
    }
}

extern "C" int vt_streams_fill(const float* h, float* x, int n, int S, int W, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && S >= 1 && W > 0, "vt_streams_fill: bad sizes n=%d S=%d W=%d", n, S, W);
    if (n == 0) return 0;
    const long long total = (long long)n * W;
    long long blocks = (total + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    streams_fill_kernel<<<(unsigned)blocks, 256, 0, stream>>>(h, x, S, W, total);
    VT_CHECK_LAUNCH("vt_streams_fill");
    return 0;
}

template <typename TO>
__global__ __launch_bounds__(256) void streams_read_kernel(const float* __restrict__ x, const float* __restrict__ w_in,
                                                           const float* __restrict__ gain, const int* __restrict__ rows,
                                                           TO* __restrict__ out, int S, int W, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int t = rows ? rows[r] : r;
    const float* xt = x + (size_t)t * S * W;
    float wi[STREAMS_MAX];
#pragma unroll
    for (int s = 0; s < STREAMS_MAX; ++s) wi[s] = s < S ? w_in[s] : 0.f;
    float ss = 0.f;
    for (int j = threadIdx.x; j < W; j += 256) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) u = fmaf(wi[s], xt[(size_t)s * W + j], u);
        ss = fmaf(u, u, ss);
    }
    ss = block_sum(ss, red);
    const float rinv = 1.0f / sqrtf(ss / (float)W + eps);
    for (int j = threadIdx.x; j < W; j += 256) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s)
            if (s < S) u = fmaf(wi[s], xt[(size_t)s * W + j], u);
        store_f32<TO>(out, (size_t)r * W + j, (gain[j] * u) * rinv);
    }
}

// The same for widths that are multiples of 4 up to 1024 NV: a thread keeps its NV pieces of four sums in registers
// between the two passes, so the streams are read once, 16 bytes at a time, with all of a thread's loads in flight
// together.  The weighted sums are those of the kernel above; the sum of squares takes its terms in this layout's order
// (which of the two kernels runs depends on the width alone).
template <typename TO, int NV>
__global__ __launch_bounds__(256) void streams_read_vec_kernel(const float* __restrict__ x, const float* __restrict__ w_in,
                                                               const float* __restrict__ gain, const int* __restrict__ rows,
                                                               TO* __restrict__ out, int S, int W, float eps) {
    __shared__ float red[16];
    const int r = blockIdx.x;
    const int t = rows ? rows[r] : r;
    const int W4 = W >> 2;
    const float4* xt = (const float4*)(x + (size_t)t * S * W);
    float4 u[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) u[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < S; ++s) {
        const float wi = w_in[s];
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int j = threadIdx.x + 256 * i;
            if (j < W4) {
                const float4 v = xt[(size_t)s * W4 + j];
                u[i].x = fmaf(wi, v.x, u[i].x);
                u[i].y = fmaf(wi, v.y, u[i].y);
                u[i].z = fmaf(wi, v.z, u[i].z);
                u[i].w = fmaf(wi, v.w, u[i].w);
            }
        }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        ss = fmaf(u[i].x, u[i].x, ss);
        ss = fmaf(u[i].y, u[i].y, ss);
        ss = fmaf(u[i].z, u[i].z, ss);
        ss = fmaf(u[i].w, u[i].w, ss);
    }
    ss = block_sum(ss, red);
    const float rinv = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int j = threadIdx.x + 256 * i;
        if (j < W4) {
            const float4 gn = ((const float4*)gain)[j];
            const float a = (gn.x * u[i].x) * rinv, b = (gn.y * u[i].y) * rinv, c = (gn.z * u[i].z) * rinv, d = (gn.w * u[i].w) * rinv;
            if constexpr (sizeof(TO) == 4) {
                ((float4*)out)[(size_t)r * W4 + j] = make_float4(a, b, c, d);
            } else {
                uint2 o;
                o.x = vt_pack2(a, b);
                o.y = vt_pack2(c, d);
                ((uint2*)out)[(size_t)r * W4 + j] = o;
            }
        }
    }
}

template <typename TO>
static void streams_read_launch(const float* x, const float* w_in, const float* gain, const int* rows, TO* out, int n_out, int S,
                                int W, float eps, hipStream_t stream) {
    const bool vec = W % 4 == 0 && W <= 8192 && !(((uintptr_t)x | (uintptr_t)gain | (uintptr_t)out) & 15);
    if (vec && W <= 1024) streams_read_vec_kernel<TO, 1><<<n_out, 256, 0, stream>>>(x, w_in, gain, rows, out, S, W, eps);
    else if (vec && W <= 2048) streams_read_vec_kernel<TO, 2><<<n_out, 256, 0, stream>>>(x, w_in, gain, rows, out, S, W, eps);
    else if (vec && W <= 4096) streams_read_vec_kernel<TO, 4><<<n_out, 256, 0, stream>>>(x, w_in, gain, rows, out, S, W, eps);
    else if (vec) streams_read_vec_kernel<TO, 8><<<n_out, 256, 0, stream>>>(x, w_in, gain, rows, out, S, W, eps);
    else streams_read_kernel<TO><<<n_out, 256, 0, stream>>>(x, w_in, gain, rows, out, S, W, eps);
}

extern "C" int vt_streams_read(const float* x, const float* w_in, const float* gain, const int* rows, void* out,
                               int out_dtype, int n_out, int S, int W, float eps, hipStream_t stream) {
    VT_REQUIRE(n_out >= 0 && W > 0, "vt_streams_read: bad sizes n=%d W=%d", n_out, W);
    VT_REQUIRE(S >= 1 && S <= STREAMS_MAX, "vt_streams_read: %d streams (1 to %d)", S, STREAMS_MAX);
    if (n_out == 0) return 0;
    if (out_dtype == VT_F32) streams_read_launch<float>(x, w_in, gain, rows, (float*)out, n_out, S, W, eps, stream);
    else if (out_dtype == VT_BF16) streams_read_launch<bf16_t>(x, w_in, gain, rows, (bf16_t*)out, n_out, S, W, eps, stream);
    else return vt_fail("vt_streams_read: unknown out dtype %d", out_dtype);
    VT_CHECK_LAUNCH("vt_streams_read");
    return 0;
}

template <typename TY, typename TG>
__global__ __launch_bounds__(256) void streams_write_kernel(float* __restrict__ x, const float* __restrict__ mix,
                                                            const float* __restrict__ w_out, const TY* __restrict__ y,
                                                            const TG* __restrict__ gate, int S, int W, long long total) {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const long long t = i / W;
        const int j = (int)(i - t * W);
        float* xt = x + (size_t)t * S * W + j;
        float v = load_f32<TY>(y, (size_t)i);
        if (gate) v = v / (1.0f + expf(-load_f32<TG>(gate, (size_t)i)));
        float old[STREAMS_MAX];
#pragma unroll
        for (int s = 0; s < STREAMS_MAX; ++s) old[s] = s < S ? xt[(size_t)s * W] : 0.f;
        for (int to = 0; to < S; ++to) {
            float acc = 0.f;
#pragma unroll
            for (int s = 0; s < STREAMS_MAX; ++s)
                if (s < S) acc = fmaf(mix[s * S + to], old[s], acc);
            xt[(size_t)to * W] = fmaf(w_out[to], v, acc);
        }
    }
}

extern "C" int vt_streams_write(float* x, const float* mix, const float* w_out, const void* y, int y_dtype, const void* gate,
                                int gate_dtype, int n, int S, int W, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && W > 0, "vt_streams_write: bad sizes n=%d W=%d", n, W);
    VT_REQUIRE(S >= 1 && S <= STREAMS_MAX, "vt_streams_write: %d streams (1 to %d)", S, STREAMS_MAX);
    if (n == 0) return 0;
    const long long total = (long long)n * W;
    long long blocks = (total + 255) / 256;
    if (blocks > 32768) blocks = 32768;
    if (!gate) gate_dtype = y_dtype;
#define VT_SW(TY, TG) streams_write_kernel<TY, TG><<<(unsigned)blocks, 256, 0, stream>>>(x, mix, w_out, (const TY*)y, (const TG*)gate, S, W, total)
    if (y_dtype == VT_F32 && gate_dtype == VT_F32) VT_SW(float, float);
    else if (y_dtype == VT_F32 && gate_dtype == VT_BF16) VT_SW(float, bf16_t);
    else if (y_dtype == VT_BF16 && gate_dtype == VT_F32) VT_SW(bf16_t, float);
    else if (y_dtype == VT_BF16 && gate_dtype == VT_BF16) VT_SW(bf16_t, bf16_t);
    else return vt_fail("vt_streams_write: dtypes %d / %d are not handled", y_dtype, gate_dtype);
#undef VT_SW
    VT_CHECK_LAUNCH("vt_streams_write");
    return 0;
}

template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                                          float* __restrict__ state, long long slot_stride,
                                                          const int* __restrict__ tok_entry, const int* __restrict__ entry_start,
                                                          const int* __restrict__ slots, T* __restrict__ out, int W) {
    const int t = blockIdx.x;
    const int j = blockIdx.y * 256 + threadIdx.x;
    if (j >= W) return;
    const int e = tok_entry[t];
    const int start = entry_start[e];
    const float cur = load_f32<T>(h, (size_t)t * W + j);
    float prev;
    if (t > start) {
        prev = load_f32<T>(h, (size_t)(t - 1) * W + j);
    } else {
        float* st = state + (size_t)slots[e] * slot_stride + j;
        prev = *st;
        *st = load_f32<T>(h, (size_t)(entry_start[e + 1] - 1) * W + j);
    }
    store_f32<T>(out, (size_t)t * W + j, fmaf(prev - cur, mu[j], cur));
}

extern "C" int vt_token_shift(const void* h, int dtype, const float* mu, float* state, long long slot_stride,
                              const int* tok_entry, const int* entry_start, const int* slots, void* out, int n, int W,
                              hipStream_t stream) {
    VT_REQUIRE(n >= 0 && W > 0 && slot_stride >= W, "vt_token_shift: bad sizes n=%d W=%d (state slots of %lld)", n, W, slot_stride);
    VT_REQUIRE(W <= 65535 * 256, "vt_token_shift: rows too wide");
    if (n == 0) return 0;
    const dim3 grid(n, (W + 255) / 256);
    if (dtype == VT_F32)
        token_shift_kernel<float><<<grid, 256, 0, stream>>>((const float*)h, mu, state, slot_stride, tok_entry, entry_start, slots, (float*)out, W);
    else if (dtype == VT_BF16)
        token_shift_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)h, mu, state, slot_stride, tok_entry, entry_start, slots, (bf16_t*)out, W);
    else return vt_fail("vt_token_shift: unknown dtype %d", dtype);
    VT_CHECK_LAUNCH("vt_token_shift");
    return 0;
}
