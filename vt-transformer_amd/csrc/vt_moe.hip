// A feed-forward made of many small gated ones ("experts"), of which a router chooses a few per token.
//
//   vt_moe_route:    logits z = W_r x in float32 (W_r is kept in float32), scores sigmoid(z) or softmax(z), the `top`
//                    largest per token (the lower index among equals), optionally divided by their sum.  A block per token.
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

// a wave's dot product of a float32 row with a float32 vector in LDS, 16 bytes per lane at a time where the row allows
__device__ __forceinline__ float wave_dot_f32(const float* __restrict__ row, const float* __restrict__ v, int K, int lane) {
    float acc = 0.f;
    if (K % 4 == 0 && !((uintptr_t)row & 15)) {
#pragma unroll 4
        for (int j = lane * 4; j < K; j += 256) {
            const float4 w = *(const float4*)(row + j);
            acc = fmaf(w.x, v[j], acc);
            acc = fmaf(w.y, v[j + 1], acc);
            acc = fmaf(w.z, v[j + 2], acc);
            acc = fmaf(w.w, v[j + 3], acc);
        }
    } else {
        for (int j = lane; j < K; j += 64) acc = fmaf(row[j], v[j], acc);
    }
    return wave_sum(acc);
}

// A block of four waves per token: the token lies in LDS as float32, the waves take the experts in turn, and the
// first wave then picks the largest scores.
template <typename TI>
__global__ __launch_bounds__(256) void moe_route_kernel(const TI* __restrict__ x, const float* __restrict__ wr,
                                                        int* __restrict__ ids, float* __restrict__ wts, int E, int W, int top,
                                                        int softmax, int renorm) {
    extern __shared__ float sh[];       // W values of the token, then E scores
    float* xs = sh;
    float* sc = sh + W;
    const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const TI* xt = x + (size_t)t * W;
    for (int j = threadIdx.x; j < W; j += 256) xs[j] = load_f32<TI>(xt, j);
    __syncthreads();
    for (int e = wave; e < E; e += 4) {
        const float acc = wave_dot_f32(wr + (size_t)e * W, xs, W, lane);
        if (lane == 0) sc[e] = acc;
    }
    __syncthreads();
    if (wave != 0) return;
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
    VT_REQUIRE(E + W <= 16000, "vt_moe_route: %d experts and a width of %d (together up to 16000)", E, W);
    if (n == 0) return 0;
    const size_t lds = (size_t)(E + W) * sizeof(float);
    if (dtype == VT_F32) moe_route_kernel<float><<<n, 256, lds, stream>>>((const float*)x, wr, ids, wts, E, W, top, softmax, renorm);
    else if (dtype == VT_BF16) moe_route_kernel<bf16_t><<<n, 256, lds, stream>>>((const bf16_t*)x, wr, ids, wts, E, W, top, softmax, renorm);
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

// ---------------------------------------------------------------------------
// Many tokens.  vt_moe_sort puts the (token, choice) pairs in the order of their experts and cuts every expert's run
// of pairs into tiles of up to 128; the two grouped products then take a tile of pairs times 128 rows of the
// expert's matrix per block on the matrix cores, so an expert's matrices are read once per 128 pairs that chose it.
// Nothing of this reaches the host: the launches are sized for the most tiles there can be (pairs / 128 + experts),
// and a block whose tile does not exist leaves at once.
//
// The plan (int32): [0] tiles in use; then order[P] (the pair at every sorted place), and per tile its expert, its
// first sorted place and its number of pairs (T entries each).  A pair's place among its expert's pairs is whatever
// the atomic counters give it: a matrix instruction's result for a row depends on that row and the matrix alone, in a
// summation order that the instruction fixes, so a token's result does not depend on its place or its neighbours.
//
// A block of four waves; a wave multiplies 64 rows of the matrix (first operand: a lane then holds four consecutive
// outputs of one pair) with 64 pairs by v_mfma_f32_16x16x32 from LDS, where both tiles lie with rows of 64 k padded
// to 72 elements, which puts the sixteen rows that a quarter of a wave reads on different banks.  Two stages in LDS;
// the next stage's pieces travel through registers while the current one is multiplied (the pairs' inputs are scaled
// by their scores on the way where the score multiplies an expert's input), one barrier per stage.
// ---------------------------------------------------------------------------
#define GR_TB 128                   // pairs per tile
#define GR_FB 128                   // rows of the expert's matrices per tile (gated: 64 gate rows and their 64 up rows)
#define GR_BK 64                    // k per stage
#define GR_LD 72                    // elements of a row in LDS
#define GR_STAGE ((GR_TB + GR_FB) * GR_LD)
#define GR_LDS_BYTES (2 * GR_STAGE * 2)
#define GR_MAX_EXPERTS 1024
#define GR_FEW_PAIRS 64             // up to so many pairs in a step the products go 16 rows of a matrix to a block

extern "C" int vt_moe_plan_tiles(int pairs, int E) { return (pairs + GR_TB - 1) / GR_TB + E; }
extern "C" long long vt_moe_plan_size(int pairs, int E) { return 1 + (long long)pairs + 3ll * vt_moe_plan_tiles(pairs, E); }

__global__ __launch_bounds__(1024) void moe_sort_kernel(const int* __restrict__ ids, int* __restrict__ plan, int P, int E, int T) {
    extern __shared__ int sm[];         // counts [E], cursors [E]
    __shared__ unsigned long long sc[1024];
    int* cnt = sm;
    int* cur = sm + E;
    int* order = plan + 1;
    int* tile_expert = order + P;
    int* tile_row0 = tile_expert + T;
    int* tile_rows = tile_row0 + T;
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 1024) cnt[e] = 0;
    __syncthreads();
    for (int p = tid; p < P; p += 1024) atomicAdd(&cnt[ids[p]], 1);
    __syncthreads();
    const int c = tid < E ? cnt[tid] : 0;
    const int tiles = (c + GR_TB - 1) / GR_TB;
    // running sums of the pairs (low word) and the tiles (high word) of the experts up to this one
    sc[tid] = ((unsigned long long)tiles << 32) | (unsigned)c;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
        const unsigned long long add = tid >= o ? sc[tid - o] : 0ull;
        __syncthreads();
        sc[tid] += add;
        __syncthreads();
    }
    const unsigned long long incl = sc[tid];
    const int off = (int)(unsigned)(incl & 0xffffffffull) - c;
    const int toff = (int)(incl >> 32) - tiles;
    if (tid < E) {
        cur[tid] = off;
        for (int i = 0; i < tiles; ++i) {
            tile_expert[toff + i] = tid;
            tile_row0[toff + i] = off + i * GR_TB;
            tile_rows[toff + i] = min(GR_TB, c - i * GR_TB);
        }
    }
    if (tid == 1023) plan[0] = (int)(incl >> 32);
    __syncthreads();
    for (int p = tid; p < P; p += 1024) order[atomicAdd(&cur[ids[p]], 1)] = p;
}

// ids [pairs] with values in [0, E); plan: vt_moe_plan_size(pairs, E) ints
extern "C" int vt_moe_sort(const int* ids, int* plan, int pairs, int E, hipStream_t stream) {
    VT_REQUIRE(pairs >= 0 && E > 0 && E <= GR_MAX_EXPERTS, "vt_moe_sort: %d pairs, %d experts (up to %d)", pairs, E, GR_MAX_EXPERTS);
    if (pairs == 0) return 0;
    moe_sort_kernel<<<1, 1024, 2 * (size_t)E * sizeof(int), stream>>>(ids, plan, pairs, E, vt_moe_plan_tiles(pairs, E));
    VT_CHECK_LAUNCH("vt_moe_sort");
    return 0;
}

struct GroupedArgs {
    const bf16_t* x;        // gated: the tokens [n][K]; else the activations in sorted order [P][K]
    const bf16_t* w;        // gated: [E][2 M][K] (gate rows, then up rows); else [E][M][K]
    const int* plan;
    const float* wts;       // the pairs' scores
    void* out;              // gated: activations in sorted order [P][M], 16 bits; else float32 [P][M] in the pairs' order
    int P, K, M, top, T, scale;
    float alpha, cubic;
};

typedef __attribute__((ext_vector_type(4))) float moe_f32x4_t;
union MoeFrag {
    uint4 u;
    vt_lowp8_t v;
};

__device__ __forceinline__ unsigned moe_scale2(unsigned u, float s) { return vt_pack2(lowp_lo(u) * s, lowp_hi(u) * s); }

template <bool GATED>
__global__ __launch_bounds__(256) void moe_grouped_kernel(GroupedArgs a) {
    const int tile = blockIdx.y;
    if (tile >= a.plan[0]) return;
    const int* order = a.plan + 1;
    const int* tile_expert = order + a.P;
    const int e = tile_expert[tile], row0 = tile_expert[a.T + tile], rows = tile_expert[2 * a.T + tile];
    extern __shared__ __attribute__((aligned(16))) bf16_t gl[];      // [2][GR_FB + GR_TB][GR_LD]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int wf = wave >> 1, wt = wave & 1;
    const int K = a.K, M = a.M;
    // a thread brings piece c (8 values) of rows lr, lr + 32, lr + 64, lr + 96 of both tiles
    const int c = tid & 7, lr = tid >> 3;
    const bf16_t* xrow[4];
    const bf16_t* wrow[4];
    float xscale[4];
    const bool scaled = GATED && a.scale;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = lr + 32 * i;
        const int rr = min(row, rows - 1);          // beyond the tile's pairs the last one again (never stored)
        if (GATED) {
            const int p = order[row0 + rr];
            xrow[i] = a.x + (size_t)(p / a.top) * K;
            xscale[i] = scaled ? a.wts[p] : 1.f;
            const int f = min((int)blockIdx.x * 64 + (row & 63), M - 1);
            wrow[i] = a.w + ((size_t)e * 2 * M + (row < 64 ? f : M + f)) * K;
        } else {
            xrow[i] = a.x + (size_t)(row0 + rr) * K;
            xscale[i] = 1.f;
            wrow[i] = a.w + ((size_t)e * M + min((int)blockIdx.x * GR_FB + row, M - 1)) * K;
        }
    }
    uint4 xr[4], wr[4];
    auto fetch = [&](int k0) __attribute__((always_inline)) {
        const int k = k0 + c * 8;
        if (k < K) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xr[i] = *(const uint4*)(xrow[i] + k);
                wr[i] = *(const uint4*)(wrow[i] + k);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                xr[i] = make_uint4(0u, 0u, 0u, 0u);
                wr[i] = make_uint4(0u, 0u, 0u, 0u);
            }
        }
    };
    auto stash = [&](int st) __attribute__((always_inline)) {
        bf16_t* ws = gl + st * GR_STAGE;
        bf16_t* xs = ws + GR_FB * GR_LD;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            uint4 v = xr[i];
            if (scaled) {
                const float s = xscale[i];
                v.x = moe_scale2(v.x, s); v.y = moe_scale2(v.y, s); v.z = moe_scale2(v.z, s); v.w = moe_scale2(v.w, s);
            }
            *(uint4*)(xs + (lr + 32 * i) * GR_LD + c * 8) = v;
            *(uint4*)(ws + (lr + 32 * i) * GR_LD + c * 8) = wr[i];
        }
    };
    moe_f32x4_t acc[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = (moe_f32x4_t){0.f, 0.f, 0.f, 0.f};
    // rows of the matrix tile that this wave multiplies: gated, 32 gate rows (j = 0, 1) and their up rows (j = 2, 3)
    int wl[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wl[j] = (GATED ? (j < 2 ? 0 : 64) + 32 * wf + 16 * (j & 1) : 64 * wf + 16 * j) + r;
    auto multiply = [&](int st) __attribute__((always_inline)) {
        const bf16_t* ws = gl + st * GR_STAGE;
        const bf16_t* xs = ws + GR_FB * GR_LD;
#pragma unroll
        for (int ks = 0; ks < GR_BK / 32; ++ks) {
            MoeFrag wfr[4], xfr[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) wfr[j].u = *(const uint4*)(ws + wl[j] * GR_LD + (4 * ks + g) * 8);
#pragma unroll
            for (int i = 0; i < 4; ++i) xfr[i].u = *(const uint4*)(xs + (64 * wt + 16 * i + r) * GR_LD + (4 * ks + g) * 8);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j][i] = VT_MFMA_16X16X32(wfr[j].v, xfr[i].v, acc[j][i]);
        }
    };
    const int stages = (K + GR_BK - 1) / GR_BK;
    fetch(0);
    stash(0);
    __syncthreads();
    for (int st = 0; st < stages; ++st) {
        if (st + 1 < stages) fetch((st + 1) * GR_BK);
        multiply(st & 1);
        if (st + 1 < stages) stash((st + 1) & 1);
        __syncthreads();
    }
    // acc[j][i][q]: row wl[j] - r + 4 g + q of the matrix tile, pair 64 wt + 16 i + r
    if (GATED) {
        bf16_t* act = (bf16_t*)a.out;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int f = (int)blockIdx.x * 64 + 32 * wf + 16 * j + 4 * g;
            if (f >= M) continue;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 64 * wt + 16 * i + r;
                if (row >= rows) continue;
                float v[4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const float gt = acc[j][i][q], up = acc[2 + j][i][q];
                    const float z = a.cubic != 0.f ? a.alpha * gt * fmaf(a.cubic * gt, gt, 1.f) : a.alpha * gt;
                    v[q] = gt / (1.0f + expf(-z)) * up;
                }
                uint2 o;
                o.x = vt_pack2(v[0], v[1]);
                o.y = vt_pack2(v[2], v[3]);
                *(uint2*)(act + (size_t)(row0 + row) * M + f) = o;
            }
        }
    } else {
        float* out = (float*)a.out;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = 64 * wt + 16 * i + r;
            if (row >= rows) continue;
            const int p = order[row0 + row];
            const float s = a.scale ? a.wts[p] : 1.f;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int m = (int)blockIdx.x * GR_FB + 64 * wf + 16 * j + 4 * g;
                if (m >= M) continue;
                float4 o;
                o.x = s * acc[j][i][0];
                o.y = s * acc[j][i][1];
                o.z = s * acc[j][i][2];
                o.w = s * acc[j][i][3];
                *(float4*)(out + (size_t)p * M + m) = o;
            }
        }
    }
}

// Few pairs (decoding): an expert's tile holds a handful of pairs, and what bounds the products is how fast the
// experts' matrices stream in.  A block takes 16 rows of the expert's matrix (gated: 16 gate rows and their up rows)
// and up to 16 pairs at a time; its four waves split K in turns of 64 (a cache line of every row) and read their
// operands straight from memory (a lane 16 bytes of its row), two turns' loads in flight; the waves' sums meet in LDS in a fixed order.  Sixteen
// rows to a block give eight times the blocks of the tiled kernel, which is what fills the GPU when the pairs are few.
template <bool GATED>
__global__ __launch_bounds__(256) void moe_few_kernel(GroupedArgs a) {
    const int tile = blockIdx.y;
    if (tile >= a.plan[0]) return;
    const int* order = a.plan + 1;
    const int* tile_expert = order + a.P;
    const int e = tile_expert[tile], row0 = tile_expert[a.T + tile], rows = tile_expert[2 * a.T + tile];
    __shared__ float red[3][GATED ? 2 : 1][4][64];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int r = lane & 15, g = lane >> 4;
    const int K = a.K, M = a.M;
    const int m0 = (int)blockIdx.x * 16;
    const int mr = min(m0 + r, M - 1);
    const bf16_t* w0 = a.w + ((size_t)e * (GATED ? 2 : 1) * M + mr) * K;
    const bf16_t* w1 = GATED ? w0 + (size_t)M * K : w0;
    const bool scaled = GATED && a.scale;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    for (int sub = 0; sub < rows; sub += 16) {
        const int pr = row0 + min(sub + r, rows - 1);       // beyond the tile's pairs the last one again (never stored)
        const bf16_t* xrow;
        float xs = 1.f;
        if (GATED) {
            const int p = order[pr];
            xrow = a.x + (size_t)(p / a.top) * K;
            if (scaled) xs = a.wts[p];
        } else {
            xrow = a.x + (size_t)pr * K;
        }
        moe_f32x4_t acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
        // a wave's turn: 64 of K, one 128-byte line of every row, as two products
#pragma unroll 2
        for (int kb = 64 * wave; kb < K; kb += 256) {
            MoeFrag wa[2], wb[2], xf[2];
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int k = kb + 32 * h + 8 * g;
                const bool in = k < K;
                wa[h].u = in ? *(const uint4*)(w0 + k) : zero;
                wb[h].u = (GATED && in) ? *(const uint4*)(w1 + k) : zero;
                xf[h].u = in ? *(const uint4*)(xrow + k) : zero;
            }
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (scaled) {
                    xf[h].u.x = moe_scale2(xf[h].u.x, xs); xf[h].u.y = moe_scale2(xf[h].u.y, xs);
                    xf[h].u.z = moe_scale2(xf[h].u.z, xs); xf[h].u.w = moe_scale2(xf[h].u.w, xs);
                }
                acc0 = VT_MFMA_16X16X32(wa[h].v, xf[h].v, acc0);
                if (GATED) acc1 = VT_MFMA_16X16X32(wb[h].v, xf[h].v, acc1);
            }
        }
        if (wave) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                red[wave - 1][0][q][lane] = acc0[q];
                if (GATED) red[wave - 1][GATED ? 1 : 0][q][lane] = acc1[q];
            }
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int v = 0; v < 3; ++v)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    acc0[q] += red[v][0][q][lane];
                    if (GATED) acc1[q] += red[v][GATED ? 1 : 0][q][lane];
                }
            // acc[q]: row m0 + 4 g + q of the expert's matrix, pair sub + r of the tile
            const int row = sub + r, m = m0 + 4 * g;
            if (row < rows && m < M) {
                if (GATED) {
                    float v4[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const float gt = acc0[q], up = acc1[q];
                        const float z = a.cubic != 0.f ? a.alpha * gt * fmaf(a.cubic * gt, gt, 1.f) : a.alpha * gt;
                        v4[q] = gt / (1.0f + expf(-z)) * up;
                    }
                    uint2 o;
                    o.x = vt_pack2(v4[0], v4[1]);
                    o.y = vt_pack2(v4[2], v4[3]);
                    *(uint2*)((bf16_t*)a.out + (size_t)(row0 + row) * M + m) = o;
                } else {
                    const int p = order[row0 + row];
                    const float s = a.scale ? a.wts[p] : 1.f;
                    *(float4*)((float*)a.out + (size_t)p * M + m) = make_float4(s * acc0[0], s * acc0[1], s * acc0[2], s * acc0[3]);
                }
            }
        }
        __syncthreads();
    }
}

// out[t] = sum of y[t * top + k] over k = 0, 1, .. in that order
__global__ __launch_bounds__(256) void moe_combine_kernel(const float* __restrict__ y, float* __restrict__ out, int W4, int top,
                                                          long long total4) {
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total4; i += (long long)gridDim.x * 256) {
        const long long t = i / W4;
        const int j = (int)(i - t * W4);
        const float4* src = (const float4*)y + (size_t)t * top * W4 + j;
        float4 s = src[0];
        for (int k = 1; k < top; ++k) {
            const float4 v = src[(size_t)k * W4];
            s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w;
        }
        ((float4*)out)[i] = s;
    }
}

static int grouped_ready() {
    static int done = 0;
    if (done) return 0;
    hipError_t e1 = hipFuncSetAttribute((const void*)moe_grouped_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, GR_LDS_BYTES);
    hipError_t e2 = hipFuncSetAttribute((const void*)moe_grouped_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, GR_LDS_BYTES);
    if (e1 != hipSuccess || e2 != hipSuccess) return vt_fail("vt_moe: the grouped products' LDS could not be set");
    done = 1;
    return 0;
}

// act (sorted order) [n * top][F] <- the gated units of every pair; x [n][W], w_gu [E][2 F][W], both of the 16-bit type
extern "C" int vt_moe_gate_up_grouped(const void* x, const void* w_gu, const int* plan, const float* wts, void* act, int n,
                                      int E, int W, int F, int top, int scale_input, float alpha, float cubic,
                                      hipStream_t stream) {
    VT_REQUIRE(n >= 0 && E > 0 && E <= GR_MAX_EXPERTS && top > 0, "vt_moe_gate_up_grouped: bad sizes");
    VT_REQUIRE(W > 0 && F > 0 && W % 8 == 0 && F % 8 == 0, "vt_moe_gate_up_grouped: width %d and experts' size %d (multiples of 8)", W, F);
    VT_REQUIRE(!(((uintptr_t)x | (uintptr_t)w_gu | (uintptr_t)act) & 15), "vt_moe_gate_up_grouped: operands must be 16-byte aligned");
    VT_REQUIRE(alpha > 0.f, "vt_moe_gate_up_grouped: bad gate");
    if (n == 0) return 0;
    if (grouped_ready()) return -1;
    const int P = n * top, T = vt_moe_plan_tiles(P, E);
    VT_REQUIRE(T <= 65535, "vt_moe_gate_up_grouped: too many pairs (%d)", P);
    GroupedArgs a = {(const bf16_t*)x, (const bf16_t*)w_gu, plan, wts, act, P, W, F, top, T, scale_input, alpha, cubic};
    if (P <= GR_FEW_PAIRS) moe_few_kernel<true><<<dim3((F + 15) / 16, T), 256, 0, stream>>>(a);
    else moe_grouped_kernel<true><<<dim3((F + 63) / 64, T), 256, GR_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_moe_gate_up_grouped");
    return 0;
}

// out [n][W] float32 <- the sum over a token's choices of W_down,e act; act (sorted order) [n * top][F], w_down [E][W][F];
// y: float32 scratch [n * top][W], needed when top > 1
extern "C" int vt_moe_down_grouped(const void* act, const void* w_down, const int* plan, const float* wts, float* out, float* y,
                                   int n, int E, int W, int F, int top, int scale_output, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && E > 0 && E <= GR_MAX_EXPERTS && top > 0, "vt_moe_down_grouped: bad sizes");
    VT_REQUIRE(W > 0 && F > 0 && W % 8 == 0 && F % 8 == 0, "vt_moe_down_grouped: width %d and experts' size %d (multiples of 8)", W, F);
    VT_REQUIRE(!(((uintptr_t)act | (uintptr_t)w_down | (uintptr_t)out | (uintptr_t)y) & 15), "vt_moe_down_grouped: operands must be 16-byte aligned");
    VT_REQUIRE(top == 1 || y, "vt_moe_down_grouped: %d choices per token need scratch", top);
    if (n == 0) return 0;
    if (grouped_ready()) return -1;
    const int P = n * top, T = vt_moe_plan_tiles(P, E);
    VT_REQUIRE(T <= 65535, "vt_moe_down_grouped: too many pairs (%d)", P);
    GroupedArgs a = {(const bf16_t*)act, (const bf16_t*)w_down, plan, wts, top == 1 ? (void*)out : (void*)y, P, F, W, top, T,
                     scale_output, 1.f, 0.f};
    if (P <= GR_FEW_PAIRS) moe_few_kernel<false><<<dim3((W + 15) / 16, T), 256, 0, stream>>>(a);
    else moe_grouped_kernel<false><<<dim3((W + GR_FB - 1) / GR_FB, T), 256, GR_LDS_BYTES, stream>>>(a);
    VT_CHECK_LAUNCH("vt_moe_down_grouped");
    if (top > 1) {
        const long long total4 = (long long)n * (W / 4);
        long long blocks = (total4 + 255) / 256;
        if (blocks > 16384) blocks = 16384;
        moe_combine_kernel<<<(unsigned)blocks, 256, 0, stream>>>(y, out, W / 4, top, total4);
        VT_CHECK_LAUNCH("vt_moe_down_grouped (sum)");
    }
    return 0;
}
