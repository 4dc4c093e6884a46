// The gated delta rule as a token mixer with per-request state, for prompts and decoding alike.
//
// Per head, a matrix state S [D][Dv] in float32 is carried from token to token:
//     S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q        (the read-out sees the token's own write)
// with q and k scaled to unit length (q also by D^-1/2), beta = sigmoid(b) and the decay
// g = exp(-exp(A_log) softplus(a + dt_bias)), all in float32.  In front of it q, k and v pass a short causal
// convolution over time per channel and a SiLU; the convolution's last taps - 1 inputs are part of the state.
//
//   vt_short_conv:        y[t][c] = silu(sum_j taps[c][j] x[t - (K-1) + j][c]); inputs before a request's first token
//                         of this step come from its state (zeros at the start of a sequence).
//   vt_short_conv_carry:  the last K-1 inputs of every request go into its state (after vt_short_conv has read it).
//   vt_delta_rule:        the recurrence.  A block takes 16 value columns of one (request, head); the 16 lanes of a
//                         row share a column, each holding a sixteenth of its D state elements in registers, and
//                         add their shares up by rotations within the row.  Tokens are taken in tiles of 16 through
//                         LDS; every token is computed by the same instructions in the same order whatever the
//                         tile, so a result does not depend on how the request was cut into steps.
//   vt_gated_rmsnorm:     out = o / rms(o) * w * silu(gate) (or sigmoid(gate)), per (token, head); w shared by the heads
//                         or one per head.
//
// The generalized delta rule beside it: a decay per key channel instead of one per head, and what is taken out of
// the state lies along the unit key, scaled per channel:
//     S <- diag(w) S - (a * u)(u^T S) + k v^T,  u = k / sqrt(|k|^2 + eps);   o = S^T r      (both terms read the old S)
// with w = exp(-c * sigmoid(z)) from decay logits z and a = sigmoid(removal logits), all in float32.
//   vt_lowrank_tanh:      z[t][j] = bias[j] + sum_l W2[j][l] tanh(x[t][l]): the decay logits from a low-rank projection
//                         (act 0: without the tanh, for low-rank projections whose middle is linear; with `a_log` the
//                         sums leave as decays, exp(-exp(a_log[head]) softplus(sum)): what a recurrence would otherwise
//                         work out token by token is computed here for all tokens at once).
//   vt_general_delta:     the recurrence, in vt_delta_rule's arrangement (a row of 16 lanes per state column).
//
// The gated delta rule with a decay per key channel (vt_delta_rule_channel): the first rule above with
//     S <- diag(g) S,   g[d] = exp(-exp(A_log[head]) softplus(z[d]))
// with the decays g [n][H * D] in float32 computed in front of it (vt_lowrank_tanh with a_log).
//
// The matrix memory of xLSTM (vt_matrix_memory): per head S [D][Dv], a normalizer n [D] and a running maximum m of
// the gates' logarithms, all float32 and all zero at the start of a sequence:
//     i = cap tanh(a_i / cap),  f = logsigmoid(cap tanh(a_f / cap))           from the gates' logits a_i, a_f
//     m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n <- e^(f + m - m') n + e^(i - m') k
//     o = S^T q / (max(|n . q|, e^(-m')) + 1e-6)
// in vt_delta_rule's arrangement; every block of 16 value columns carries n and m for itself (they are kept once
// per block of columns in the state, so that no block reads what another has already moved on).
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// ---------------------------------------------------------------------------
struct ConvArgs {
    const void* x;          // [n][ldx], channels 0..C-1
    const float* taps;      // [C][K]
    float* state;           // slot s: state + s * slot_stride, [K-1][C]
    const int* tok_entry;
    const int* entry_start; // [entries + 1]
    const int* slots;
    void* y;                // [n][C]
    long long ldx, slot_stride;
    int C, K, n_entries;
};

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void short_conv_kernel(ConvArgs a) {
    const int t = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int e = a.tok_entry[t];
    const int start = a.entry_start[e];
    const float* st = a.state + (size_t)a.slots[e] * a.slot_stride;
    const int K = a.K;
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {
        const int tau = t - (K - 1) + j;
        const float v = tau >= start ? load_f32<TI>((const TI*)a.x, (size_t)tau * a.ldx + c)
                                     : st[(size_t)(K - 1 + tau - start) * a.C + c];
        acc = fmaf(a.taps[(size_t)c * K + j], v, acc);
    }
    store_f32<TO>((TO*)a.y, (size_t)t * a.C + c, silu_f(acc));
}

#define CONV_MAX_TAPS 16

template <typename TI>
__global__ __launch_bounds__(256) void short_conv_carry_kernel(ConvArgs a) {
    const int e = blockIdx.x;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int start = a.entry_start[e], end = a.entry_start[e + 1];
    float* st = a.state + (size_t)a.slots[e] * a.slot_stride;
    const int keep = a.K - 1;
    float v[CONV_MAX_TAPS];
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS; ++i) {
        if (i < keep) {
            const int tau = end - keep + i;
            v[i] = tau >= start ? load_f32<TI>((const TI*)a.x, (size_t)tau * a.ldx + c)
                                : st[(size_t)(keep + tau - start) * a.C + c];
        }
    }
#pragma unroll
    for (int i = 0; i < CONV_MAX_TAPS; ++i)
        if (i < keep) st[(size_t)i * a.C + c] = v[i];
}

static int conv_args(ConvArgs& a, const void* x, long long ldx, const float* taps, float* state, long long slot_stride,
                     const int* tok_entry, const int* entry_start, const int* slots, void* y, int n, int n_entries, int C,
                     int K, const char* who) {
    VT_REQUIRE(n >= 0 && n_entries >= 0 && C > 0, "%s: bad sizes", who);
    VT_REQUIRE(K >= 1 && K <= CONV_MAX_TAPS, "%s: %d taps (1 to %d)", who, K, CONV_MAX_TAPS);
    VT_REQUIRE(ldx >= C && slot_stride >= (long long)(K - 1) * C, "%s: rows or state slots are too short", who);
    a.x = x; a.taps = taps; a.state = state; a.tok_entry = tok_entry; a.entry_start = entry_start; a.slots = slots; a.y = y;
    a.ldx = ldx; a.slot_stride = slot_stride; a.C = C; a.K = K; a.n_entries = n_entries;
    return 0;
}

extern "C" int vt_short_conv(const void* x, int x_dtype, long long ldx, const float* taps, float* state,
                             long long slot_stride, const int* tok_entry, const int* entry_start, const int* slots,
                             void* y, int y_dtype, int n, int n_entries, int C, int K, hipStream_t stream) {
    ConvArgs a;
    if (conv_args(a, x, ldx, taps, state, slot_stride, tok_entry, entry_start, slots, y, n, n_entries, C, K, "vt_short_conv"))
        return -1;
    VT_REQUIRE(C <= 65535 * 256, "vt_short_conv: too many channels");
    if (n == 0) return 0;
    const dim3 grid(n, (C + 255) / 256);
    if (x_dtype == VT_F32 && y_dtype == VT_F32) short_conv_kernel<float, float><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_F32 && y_dtype == VT_BF16) short_conv_kernel<float, bf16_t><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_BF16 && y_dtype == VT_BF16) short_conv_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_BF16 && y_dtype == VT_F32) short_conv_kernel<bf16_t, float><<<grid, 256, 0, stream>>>(a);
    else return vt_fail("vt_short_conv: dtypes %d -> %d are not handled", x_dtype, y_dtype);
    VT_CHECK_LAUNCH("vt_short_conv");
    return 0;
}

extern "C" int vt_short_conv_carry(const void* x, int x_dtype, long long ldx, float* state, long long slot_stride,
                                   const int* entry_start, const int* slots, int n_entries, int C, int K,
                                   hipStream_t stream) {
    ConvArgs a;
    if (conv_args(a, x, ldx, nullptr, state, slot_stride, nullptr, entry_start, slots, nullptr, 0, n_entries, C, K,
                  "vt_short_conv_carry"))
        return -1;
    if (n_entries == 0 || K == 1) return 0;
    VT_REQUIRE(C <= 65535 * 256, "vt_short_conv_carry: too many channels");
    const dim3 grid(n_entries, (C + 255) / 256);
    if (x_dtype == VT_F32) short_conv_carry_kernel<float><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_BF16) short_conv_carry_kernel<bf16_t><<<grid, 256, 0, stream>>>(a);
    else return vt_fail("vt_short_conv_carry: unknown dtype %d", x_dtype);
    VT_CHECK_LAUNCH("vt_short_conv_carry");
    return 0;
}

// ---------------------------------------------------------------------------
struct DeltaArgs {
    const void* qkv;        // [n][C]: q (G x D), k (G x D), v (H x Dv), after convolution and SiLU
    const void* ba;         // ba[t * ldba + h]: beta logits, then (from column H) decay logits
    const float* a_log;     // [H]
    const float* dt_bias;   // [H]
    float* state;           // slot s: state + s * slot_stride, [H][Dv][D]
    const int* entry_start;
    const int* slots;
    float* o;               // [n][H][Dv]
    long long slot_stride, ldba;
    int H, G, D, Dv;
};

#define DELTA_TILE 16
#define DELTA_GROUPS 16     // column groups of a block: 16 lanes each

// the sum of v over the 16 lanes of a row (lanes 16 r .. 16 r + 15), in every one of them: four rotations within the row
__device__ __forceinline__ float row16_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
    return v;
}

// DS: state elements per lane and column (a sixteenth of D, rounded up to a power of two); CPL: columns per lane.
// A row of 16 lanes shares CPL value columns; lane r holds the elements d = 16 i + r, i < DS, of each: a row reads 16
// consecutive floats of LDS or of the state at a time, what it reads of k and q serves all its columns, and the
// columns' sums are chains of additions that do not wait for each other.
// The block's 256 threads are 16 rows of lanes for the recurrence and 16 tokens x 16 lanes for a tile's inputs:
// thread (tt, r) brings token tt's q and k elements 16 i + r, CPL of its values, and its gate and decay; a tile's
// inputs are asked for from memory before the recurrence over the tile in front of it starts.
template <typename TI, typename TB, int DS, int CPL>
__global__ __launch_bounds__(256) void delta_rule_kernel(DeltaArgs a) {
    constexpr int DP = 16 * DS;                       // D padded
    constexpr int COLS = DELTA_GROUPS * CPL;          // columns of a block
    __shared__ float qs[DELTA_TILE][DP];
    __shared__ float ks[DELTA_TILE][DP];
    __shared__ float vs[DELTA_TILE][COLS];
    __shared__ float beta_s[DELTA_TILE], g_s[DELTA_TILE], rq_s[DELTA_TILE], rk_s[DELTA_TILE];

    const int e = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * COLS;
    const int tid = threadIdx.x;
    const int r = tid & 15, cl = tid >> 4;
    const int D = a.D, Dv = a.Dv, H = a.H, G = a.G;
    const int kh = h / (H / G);
    const int C = 2 * G * D + H * Dv;
    const int start = a.entry_start[e], end = a.entry_start[e + 1];
    // the state of a head is kept [Dv][D]: a column's D elements lie together
    float* S_head = a.state + (size_t)a.slots[e] * a.slot_stride + (size_t)h * Dv * D;
    const TI* x = (const TI*)a.qkv;
    const TB* ba = (const TB*)a.ba;
    const float decay_rate = expf(a.a_log[h]);
    const float bias = a.dt_bias[h];
    const float q_scale = 1.0f / sqrtf((float)D);

    float S[CPL][DS];
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int col = col0 + cl * CPL + c;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = 16 * i + r;
            S[c][i] = (col < Dv && d < D) ? S_head[(size_t)col * D + d] : 0.f;
        }
    }

    // a tile's inputs in registers, as thread (tt = cl, r) brings them
    float in_q[DS], in_k[DS], in_v[CPL], in_b = 0.f, in_a = 0.f;
    auto fetch = [&](int t0) {
        const int t = t0 + cl;
        const bool ok = t < end;
        const size_t row = (size_t)(ok ? t : start) * C;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = 16 * i + r;
            const bool in = ok && d < D;
            in_q[i] = in ? load_f32<TI>(x, row + (size_t)kh * D + d) : 0.f;
            in_k[i] = in ? load_f32<TI>(x, row + (size_t)(G + kh) * D + d) : 0.f;
        }
#pragma unroll
        for (int c = 0; c < CPL; ++c) {
            const int j = col0 + r * CPL + c;
            in_v[c] = (ok && j < Dv) ? load_f32<TI>(x, row + (size_t)2 * G * D + (size_t)h * Dv + j) : 0.f;
        }
        if (r == 0 && ok) {
            in_b = load_f32<TB>(ba, (size_t)t * a.ldba + h);
            in_a = load_f32<TB>(ba, (size_t)t * a.ldba + H + h);
        }
    };
    fetch(start);
    for (int t0 = start; t0 < end; t0 += DELTA_TILE) {
        const int nt = min(DELTA_TILE, end - t0);
        __syncthreads();        // the tile before has been read
        {
            // lengths of q and k (each lane's share, then the row's sum: the same order for every token), gate and
            // decay of token cl, all in float32
            float sq = 0.f, sk = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                qs[cl][16 * i + r] = in_q[i];
                ks[cl][16 * i + r] = in_k[i];
                sq = fmaf(in_q[i], in_q[i], sq);
                sk = fmaf(in_k[i], in_k[i], sk);
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) vs[cl][r * CPL + c] = in_v[c];
            sq = row16_sum(sq);
            sk = row16_sum(sk);
            if (r == 0) {
                rq_s[cl] = q_scale / sqrtf(sq + 1e-6f);
                rk_s[cl] = 1.0f / sqrtf(sk + 1e-6f);
                beta_s[cl] = 1.0f / (1.0f + expf(-in_b));
                g_s[cl] = expf(-decay_rate * softplus_f(in_a + bias));
            }
        }
        __syncthreads();
        if (t0 + DELTA_TILE < end) fetch(t0 + DELTA_TILE);      // on its way while this tile is worked through
        // with k' = rk k and q' = rq q:  S <- g S;  u = beta (v - k'.S);  S <- S + k' u;  o = q'.S
        auto token = [&](int tt) {
            const float g = g_s[tt], beta = beta_s[tt], rq = rq_s[tt], rk = rk_s[tt];
            float kk[DS], qq[DS];
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                kk[i] = ks[tt][16 * i + r];
                qq[i] = qs[tt][16 * i + r];
            }
            float dot[CPL], out[CPL];
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DS; ++i) {
                    S[c][i] *= g;
                    acc = fmaf(kk[i], S[c][i], acc);
                }
                dot[c] = acc;
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) dot[c] = row16_sum(dot[c]);
#pragma unroll
            for (int c = 0; c < CPL; ++c) {
                const float u = beta * (vs[tt][cl * CPL + c] - rk * dot[c]) * rk;
                float acc = 0.f;
#pragma unroll
                for (int i = 0; i < DS; ++i) {
                    S[c][i] = fmaf(kk[i], u, S[c][i]);
                    acc = fmaf(qq[i], S[c][i], acc);
                }
                out[c] = acc;
            }
#pragma unroll
            for (int c = 0; c < CPL; ++c) out[c] = row16_sum(out[c]);
            if (r == 0) {
                float* o = a.o + ((size_t)(t0 + tt) * H + h) * Dv;
#pragma unroll
                for (int c = 0; c < CPL; ++c) {
                    const int col = col0 + cl * CPL + c;
                    if (col < Dv) o[col] = rq * out[c];
                }
            }
        };
        if (nt == DELTA_TILE) {
            // a whole tile as one stretch of code: a token's read-out and the next token's sums do not wait for each
            // other, and what they read from LDS is asked for early
#pragma unroll
            for (int tt = 0; tt < DELTA_TILE; ++tt) token(tt);
        } else {
            for (int tt = 0; tt < nt; ++tt) token(tt);
        }
    }
#pragma unroll
    for (int c = 0; c < CPL; ++c) {
        const int col = col0 + cl * CPL + c;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = 16 * i + r;
            if (col < Dv && d < D) S_head[(size_t)col * D + d] = S[c][i];
        }
    }
}

extern "C" int vt_delta_rule(const void* qkv, int dtype, const void* ba, int ba_dtype, long long ldba, const float* a_log,
                             const float* dt_bias, float* state, long long slot_stride, const int* entry_start,
                             const int* slots, float* o, int n_entries, int H, int G, int D, int Dv, hipStream_t stream) {
    VT_REQUIRE(n_entries >= 0 && H > 0 && G > 0 && H % G == 0, "vt_delta_rule: bad heads %d/%d", H, G);
    VT_REQUIRE(D > 0 && D <= 256 && Dv > 0, "vt_delta_rule: head sizes %d/%d (keys up to 256)", D, Dv);
    VT_REQUIRE(slot_stride >= (long long)H * D * Dv, "vt_delta_rule: state slots are too short");
    VT_REQUIRE(ldba >= 2 * H, "vt_delta_rule: rows of gate and decay logits are too short");
    VT_REQUIRE(H <= 65535, "vt_delta_rule: too many heads (%d)", H);
    if (n_entries == 0) return 0;
    DeltaArgs a;
    a.qkv = qkv; a.ba = ba; a.a_log = a_log; a.dt_bias = dt_bias; a.state = state; a.entry_start = entry_start;
    a.slots = slots; a.o = o; a.slot_stride = slot_stride; a.ldba = ldba; a.H = H; a.G = G; a.D = D; a.Dv = Dv;
    // One column to a row of lanes.  (The kernel also takes CPL = 4, four columns to a row, which shares what a row
    // reads of k and q among them; measured at 16 heads of 128 x 128 it was no faster with eight requests and half
    // again slower with one: a lone wave per SIMD issues its longer stream no faster.)
    constexpr int cpl = 1;
    const int share = (D + 15) / 16;
    const int cols = DELTA_GROUPS * cpl;
    const dim3 grid(n_entries, H, (Dv + cols - 1) / cols);
#define VT_DELTA(TI, TB)                                                                           \
    do {                                                                                           \
        if (share <= 1) delta_rule_kernel<TI, TB, 1, cpl><<<grid, 256, 0, stream>>>(a);            \
        else if (share <= 2) delta_rule_kernel<TI, TB, 2, cpl><<<grid, 256, 0, stream>>>(a);       \
        else if (share <= 4) delta_rule_kernel<TI, TB, 4, cpl><<<grid, 256, 0, stream>>>(a);       \
        else if (share <= 8) delta_rule_kernel<TI, TB, 8, cpl><<<grid, 256, 0, stream>>>(a);       \
        else delta_rule_kernel<TI, TB, 16, cpl><<<grid, 256, 0, stream>>>(a);                      \
    } while (0)
    if (dtype == VT_F32 && ba_dtype == VT_F32) VT_DELTA(float, float);
    else if (dtype == VT_BF16 && ba_dtype == VT_F32) VT_DELTA(bf16_t, float);
    else if (dtype == VT_BF16 && ba_dtype == VT_BF16) VT_DELTA(bf16_t, bf16_t);
    else return vt_fail("vt_delta_rule: dtypes %d / %d are not handled", dtype, ba_dtype);
#undef VT_DELTA
    VT_CHECK_LAUNCH("vt_delta_rule");
    return 0;
}

// ---------------------------------------------------------------------------
// out[t][h][:] = o[t][h][:] / sqrt(mean(o^2) + eps) * w[h * w_stride + :] * act(gate[t][h][:]); gate[t * ldg + h * Dv + j];
// act: silu (gate_kind 0) or sigmoid (1); w_stride 0: one weight vector for all heads, Dv: one per head
template <typename TG, typename TO>
__global__ __launch_bounds__(64) void gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                           const TG* __restrict__ gate, long long ldg, TO* __restrict__ out,
                                                           int H, int Dv, float eps, int w_stride, int gate_kind) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const float* row = o + ((size_t)t * H + h) * Dv;
    const float* wh = w + (size_t)h * w_stride;
    float ss = 0.f;
    for (int j = lane; j < Dv; j += 64) ss = fmaf(row[j], row[j], ss);
    ss = wave_sum(ss);
    const float rinv = 1.0f / sqrtf(ss / (float)Dv + eps);
    for (int j = lane; j < Dv; j += 64) {
        const float z = load_f32<TG>(gate, (size_t)t * ldg + (size_t)h * Dv + j);
        const float g = gate_kind ? 1.0f / (1.0f + expf(-z)) : silu_f(z);
        store_f32<TO>(out, ((size_t)t * H + h) * Dv + j, row[j] * rinv * wh[j] * g);
    }
}

extern "C" int vt_gated_rmsnorm(const float* o, const float* w, const void* gate, int gate_dtype, long long ldg, void* out,
                                int out_dtype, int n, int H, int Dv, float eps, int w_per_head, int gate_kind,
                                hipStream_t stream) {
    VT_REQUIRE(n >= 0 && H > 0 && Dv > 0 && H <= 65535, "vt_gated_rmsnorm: bad sizes");
    VT_REQUIRE(ldg >= (long long)H * Dv, "vt_gated_rmsnorm: gate rows are too short");
    VT_REQUIRE(gate_kind == 0 || gate_kind == 1, "vt_gated_rmsnorm: gate kind %d (0: silu, 1: sigmoid)", gate_kind);
    if (n == 0) return 0;
    const dim3 grid(n, H);
    const int ws = w_per_head ? Dv : 0;
    if (gate_dtype == VT_F32 && out_dtype == VT_F32)
        gated_rmsnorm_kernel<float, float><<<grid, 64, 0, stream>>>(o, w, (const float*)gate, ldg, (float*)out, H, Dv, eps, ws, gate_kind);
    else if (gate_dtype == VT_F32 && out_dtype == VT_BF16)
        gated_rmsnorm_kernel<float, bf16_t><<<grid, 64, 0, stream>>>(o, w, (const float*)gate, ldg, (bf16_t*)out, H, Dv, eps, ws, gate_kind);
    else if (gate_dtype == VT_BF16 && out_dtype == VT_BF16)
        gated_rmsnorm_kernel<bf16_t, bf16_t><<<grid, 64, 0, stream>>>(o, w, (const bf16_t*)gate, ldg, (bf16_t*)out, H, Dv, eps, ws, gate_kind);
    else return vt_fail("vt_gated_rmsnorm: dtypes %d -> %d are not handled", gate_dtype, out_dtype);
    VT_CHECK_LAUNCH("vt_gated_rmsnorm");
    return 0;
}

// ---------------------------------------------------------------------------
// z[t][j] = bias[j] + sum_l W2[j][l] * tanh(x[t * ldx + l]), l = 0, 1, .. in that order, float32
// A block takes TB tokens and 256 outputs: a thread reads its row of W2 once for all of them (the rows of neighbouring
// threads lie L elements apart, so each read of W2 touches as many cache lines as the wave has lanes: with many tokens
// it is what the kernel waits for, and TB tokens share it).  The sums add up in the order of l whatever TB.
template <typename TI, typename TW, int TB>
__global__ __launch_bounds__(256) void lowrank_tanh_kernel(const TI* __restrict__ x, long long ldx, const TW* __restrict__ w2,
                                                           const float* __restrict__ bias, float* __restrict__ z, int n, int L,
                                                           int M, int act, const float* __restrict__ a_log, int per_head) {
    extern __shared__ float th[];       // [TB][L]
    const int t0 = blockIdx.x * TB;
    for (int i = threadIdx.x; i < TB * L; i += 256) {
        const int tb = i / L, l = i - tb * L;
        const float v = t0 + tb < n ? load_f32<TI>(x, (size_t)(t0 + tb) * ldx + l) : 0.f;
        th[i] = act ? tanhf(v) : v;
    }
    __syncthreads();
    const int j = blockIdx.y * 256 + threadIdx.x;
    if (j >= M) return;
    float acc[TB];
    const float b0 = bias ? bias[j] : 0.f;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) acc[tb] = b0;
    for (int l = 0; l < L; ++l) {
        const float w = load_f32<TW>(w2, (size_t)j * L + l);
#pragma unroll
        for (int tb = 0; tb < TB; ++tb) acc[tb] = fmaf(w, th[tb * L + l], acc[tb]);
    }
    // the sums as decay logits: out = exp(-exp(a_log[head]) * softplus(sum)), a head being `per_head` outputs
    const float rate = a_log ? expf(a_log[j / per_head]) : 0.f;
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
        if (t0 + tb >= n) break;
        z[(size_t)(t0 + tb) * M + j] = a_log ? expf(-rate * softplus_f(acc[tb])) : acc[tb];
    }
}

extern "C" int vt_lowrank_tanh(const void* x, int x_dtype, long long ldx, const void* w2, int w_dtype, const float* bias,
                               float* z, int n, int L, int M, int act, const float* a_log, int per_head,
                               hipStream_t stream) {
    VT_REQUIRE(n >= 0 && L > 0 && L <= 8192 && M > 0 && ldx >= L, "vt_lowrank_tanh: bad sizes n=%d L=%d M=%d", n, L, M);
    VT_REQUIRE(act == 0 || act == 1, "vt_lowrank_tanh: act %d (0: none, 1: tanh)", act);
    VT_REQUIRE(!a_log || (per_head > 0 && M % per_head == 0), "vt_lowrank_tanh: %d outputs in heads of %d", M, per_head);
    VT_REQUIRE(M <= 65535 * 256, "vt_lowrank_tanh: too many outputs");
    if (n == 0) return 0;
    // many tokens and a short middle: eight tokens to a block
    const bool many = n >= 256 && L <= 1024;
    const int tb = many ? 8 : 1;
    const dim3 grid((n + tb - 1) / tb, (M + 255) / 256);
    const size_t lds = (size_t)tb * L * sizeof(float);
#define VT_LOWRANK(TI, TW)                                                                                                  \
    do {                                                                                                                    \
        if (many) lowrank_tanh_kernel<TI, TW, 8><<<grid, 256, lds, stream>>>((const TI*)x, ldx, (const TW*)w2, bias, z, n, L, M, act, a_log, per_head); \
        else lowrank_tanh_kernel<TI, TW, 1><<<grid, 256, lds, stream>>>((const TI*)x, ldx, (const TW*)w2, bias, z, n, L, M, act, a_log, per_head);      \
    } while (0)
    if (x_dtype == VT_F32 && w_dtype == VT_F32) VT_LOWRANK(float, float);
    else if (x_dtype == VT_F32 && w_dtype == VT_BF16) VT_LOWRANK(float, bf16_t);
    else if (x_dtype == VT_BF16 && w_dtype == VT_BF16) VT_LOWRANK(bf16_t, bf16_t);
    else return vt_fail("vt_lowrank_tanh: dtypes %d / %d are not handled", x_dtype, w_dtype);
#undef VT_LOWRANK
    VT_CHECK_LAUNCH("vt_lowrank_tanh");
    return 0;
}

// ---------------------------------------------------------------------------
struct GeneralDeltaArgs {
    const void* x;          // [n][ldx]: per head D read-out elements from column r_col, D keys from k_col, Dv values
                            // from v_col, D removal logits from a_col (heads one behind the other)
    const float* z;         // [n][H * D] decay logits, float32
    const float* a_bias;    // [H * D] or null: added to the removal logits
    float* state;           // slot s: state + s * slot_stride, [H][Dv][D]
    const int* entry_start;
    const int* slots;
    float* o;               // [n][H][Dv]
    long long ldx, slot_stride;
    int r_col, k_col, v_col, a_col;
    int H, D, Dv;
    float decay_scale, key_eps;
};

// vt_delta_rule's arrangement: the block's 256 threads are 16 rows of lanes for the recurrence (a row per value
// column, lane r holding the DS consecutive state elements from d = DS r, so that a token's vectors come out of LDS
// 16 bytes at a time) and TILE tokens x 16 lanes for a tile's inputs, which are
// asked for before the recurrence over the tile in front starts.  Per token and column:
//     p = u . S;   S_d <- w_d S_d - (a_d u_d) p + k_d v;   o = r . S
// the same instructions in the same order whatever the tile, so nothing depends on how a request was cut.
template <typename TI, int DS, int TILE>
__global__ __launch_bounds__(256) void general_delta_kernel(GeneralDeltaArgs a) {
    constexpr int DP = 16 * DS;
    __shared__ __attribute__((aligned(16))) float rs[TILE][DP];      // read-out vectors
    __shared__ __attribute__((aligned(16))) float ks[TILE][DP];      // keys as they come
    __shared__ __attribute__((aligned(16))) float us[TILE][DP];      // unit keys
    __shared__ __attribute__((aligned(16))) float bs[TILE][DP];      // removal rate times unit key
    __shared__ __attribute__((aligned(16))) float ws[TILE][DP];      // decays
    __shared__ float vs[TILE][DELTA_GROUPS];

    const int e = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * DELTA_GROUPS;
    const int tid = threadIdx.x;
    const int r = tid & 15, cl = tid >> 4;
    const int D = a.D, Dv = a.Dv, H = a.H;
    const int start = a.entry_start[e], end = a.entry_start[e + 1];
    float* S_head = a.state + (size_t)a.slots[e] * a.slot_stride + (size_t)h * Dv * D;
    const TI* x = (const TI*)a.x;
    const int col = col0 + cl;

    float S[DS];
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = DS * r + i;
        S[i] = (col < Dv && d < D) ? S_head[(size_t)col * D + d] : 0.f;
    }
    float ab[DS];
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = DS * r + i;
        ab[i] = (a.a_bias && d < D) ? a.a_bias[(size_t)h * D + d] : 0.f;
    }

    float in_r[DS], in_k[DS], in_a[DS], in_z[DS], in_v = 0.f;
    auto fetch = [&](int t0) {
        const int t = t0 + cl;
        const bool ok = cl < TILE && t < end;
        const size_t row = (size_t)(ok ? t : start) * a.ldx;
        const size_t zrow = (size_t)(ok ? t : start) * H * D + (size_t)h * D;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = DS * r + i;
            const bool in = ok && d < D;
            in_r[i] = in ? load_f32<TI>(x, row + a.r_col + (size_t)h * D + d) : 0.f;
            in_k[i] = in ? load_f32<TI>(x, row + a.k_col + (size_t)h * D + d) : 0.f;
            in_a[i] = in ? load_f32<TI>(x, row + a.a_col + (size_t)h * D + d) : 0.f;
            in_z[i] = in ? a.z[zrow + d] : 0.f;
        }
        const int j = col0 + r;
        in_v = (ok && j < Dv) ? load_f32<TI>(x, row + a.v_col + (size_t)h * Dv + j) : 0.f;
    };
    fetch(start);
    for (int t0 = start; t0 < end; t0 += TILE) {
        const int nt = min(TILE, end - t0);
        __syncthreads();        // the tile before has been read
        if (cl < TILE) {
            float sk = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) sk = fmaf(in_k[i], in_k[i], sk);
            sk = row16_sum(sk);
            const float rk = 1.0f / sqrtf(sk + a.key_eps);
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = DS * r + i;
                const float u = in_k[i] * rk;
                const float rate = 1.0f / (1.0f + expf(-(in_a[i] + ab[i])));
                rs[cl][d] = in_r[i];
                ks[cl][d] = in_k[i];
                us[cl][d] = u;
                bs[cl][d] = rate * u;
                ws[cl][d] = expf(-a.decay_scale / (1.0f + expf(-in_z[i])));
            }
            vs[cl][r] = in_v;
        }
        __syncthreads();
        if (t0 + TILE < end) fetch(t0 + TILE);      // on its way while this tile is worked through
        auto token = [&](int tt) {
            float p = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) p = fmaf(us[tt][DS * r + i], S[i], p);
            p = row16_sum(p);
            const float v = vs[tt][cl];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = DS * r + i;
                S[i] = fmaf(ws[tt][d], S[i], fmaf(-bs[tt][d], p, ks[tt][d] * v));
                acc = fmaf(rs[tt][d], S[i], acc);
            }
            acc = row16_sum(acc);
            if (r == 0 && col < Dv) a.o[((size_t)(t0 + tt) * H + h) * Dv + col] = acc;
        };
        if (nt == TILE) {
#pragma unroll
            for (int tt = 0; tt < TILE; ++tt) token(tt);
        } else {
            for (int tt = 0; tt < nt; ++tt) token(tt);
        }
    }
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = DS * r + i;
        if (col < Dv && d < D) S_head[(size_t)col * D + d] = S[i];
    }
}

extern "C" int vt_general_delta(const void* x, int dtype, long long ldx, int r_col, int k_col, int v_col, int a_col,
                                const float* z, const float* a_bias, float* state, long long slot_stride,
                                const int* entry_start, const int* slots, float* o, int n_entries, int H, int D, int Dv,
                                float decay_scale, float key_eps, hipStream_t stream) {
    VT_REQUIRE(n_entries >= 0 && H > 0 && H <= 65535, "vt_general_delta: bad heads %d", H);
    VT_REQUIRE(D > 0 && D <= 256 && Dv > 0, "vt_general_delta: head sizes %d/%d (keys up to 256)", D, Dv);
    VT_REQUIRE(slot_stride >= (long long)H * D * Dv, "vt_general_delta: state slots are too short");
    VT_REQUIRE(min(min(r_col, k_col), min(v_col, a_col)) >= 0 && ldx >= max(max(r_col, k_col), a_col) + (long long)H * D &&
               ldx >= v_col + (long long)H * Dv, "vt_general_delta: rows are too short for their columns");
    VT_REQUIRE(decay_scale > 0.f && key_eps >= 0.f, "vt_general_delta: bad constants");
    if (n_entries == 0) return 0;
    GeneralDeltaArgs a;
    a.x = x; a.z = z; a.a_bias = a_bias; a.state = state; a.entry_start = entry_start; a.slots = slots; a.o = o;
    a.ldx = ldx; a.slot_stride = slot_stride; a.r_col = r_col; a.k_col = k_col; a.v_col = v_col; a.a_col = a_col;
    a.H = H; a.D = D; a.Dv = Dv; a.decay_scale = decay_scale; a.key_eps = key_eps;
    const int share = (D + 15) / 16;
    const dim3 grid(n_entries, H, (Dv + DELTA_GROUPS - 1) / DELTA_GROUPS);
#define VT_GDELTA(TI)                                                                              \
    do {                                                                                           \
        if (share <= 1) general_delta_kernel<TI, 1, 16><<<grid, 256, 0, stream>>>(a);              \
        else if (share <= 2) general_delta_kernel<TI, 2, 16><<<grid, 256, 0, stream>>>(a);         \
        else if (share <= 4) general_delta_kernel<TI, 4, 16><<<grid, 256, 0, stream>>>(a);         \
        else if (share <= 8) general_delta_kernel<TI, 8, 16><<<grid, 256, 0, stream>>>(a);         \
        else general_delta_kernel<TI, 16, 8><<<grid, 256, 0, stream>>>(a);                         \
    } while (0)
    if (dtype == VT_F32) VT_GDELTA(float);
    else if (dtype == VT_BF16) VT_GDELTA(bf16_t);
    else return vt_fail("vt_general_delta: unknown dtype %d", dtype);
#undef VT_GDELTA
    VT_CHECK_LAUNCH("vt_general_delta");
    return 0;
}

// ---------------------------------------------------------------------------
// Which state element lane r (of a row of 16) holds as its i-th: groups of four consecutive elements, the groups dealt
// out to the lanes in turn (element 4 (r + 16 j) + e for i = 4 j + e), so that a row of lanes reads 256 consecutive bytes
// of the state or of a token's vectors with every 16-byte access; heads of up to 32 elements: DS consecutive ones.
template <int DS>
__device__ __forceinline__ constexpr int lane_elem(int r, int i) {
    return DS <= 4 ? DS * r + i : 4 * (r + 16 * (i / 4)) + (i % 4);
}

struct ChannelDeltaArgs {
    const void* qkv;        // [n][C]: q (G x D), k (G x D), v (H x Dv), after convolution and SiLU
    const void* beta;       // beta[t * ldb + h]: logits of the write strength
    const float* g;         // [n][H * D] decays, float32
    float* state;           // slot s: state + s * slot_stride, [H][Dv][D]
    const int* entry_start;
    const int* slots;
    float* o;               // [n][H][Dv]
    long long slot_stride, ldb;
    int H, G, D, Dv;
};

// vt_general_delta's arrangement: 16 rows of lanes for the recurrence (a row per value column, lane r holding DS state
// elements in groups of four: lane_elem) and TILE tokens x 16 lanes for a tile's inputs.  Per token and column, with
// k' and q' the unit vectors (q' also times D^-1/2):
//     S_d <- g_d S_d;  p = k' . S;  u = beta (v - p);  S_d <- S_d + k'_d u;  o = q' . S
// the same instructions in the same order whatever the tile, so nothing depends on how a request was cut.
template <typename TI, typename TB, int DS, int TILE>
__global__ __launch_bounds__(256) void delta_rule_channel_kernel(ChannelDeltaArgs a) {
    constexpr int DP = 16 * DS;
    __shared__ __attribute__((aligned(16))) float qs[TILE][DP];      // unit queries times D^-1/2
    __shared__ __attribute__((aligned(16))) float ks[TILE][DP];      // unit keys
    __shared__ __attribute__((aligned(16))) float gs[TILE][DP];      // decays
    __shared__ float vs[TILE][DELTA_GROUPS];
    __shared__ float beta_s[TILE];

    const int e = blockIdx.x, h = blockIdx.y, col0 = blockIdx.z * DELTA_GROUPS;
    const int tid = threadIdx.x;
    const int r = tid & 15, cl = tid >> 4;
    const int D = a.D, Dv = a.Dv, H = a.H, G = a.G;
    const int kh = h / (H / G);
    const int C = 2 * G * D + H * Dv;
    const int start = a.entry_start[e], end = a.entry_start[e + 1];
    float* S_head = a.state + (size_t)a.slots[e] * a.slot_stride + (size_t)h * Dv * D;
    const TI* x = (const TI*)a.qkv;
    const TB* bl = (const TB*)a.beta;
    const int col = col0 + cl;
    const float q_scale = 1.0f / sqrtf((float)D);

    float S[DS];
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = lane_elem<DS>(r, i);
        S[i] = (col < Dv && d < D) ? S_head[(size_t)col * D + d] : 0.f;
    }

    float in_q[DS], in_k[DS], in_z[DS], in_v = 0.f, in_b = 0.f;
    auto fetch = [&](int t0) {
        const int t = t0 + cl;
        const bool ok = cl < TILE && t < end;
        const size_t row = (size_t)(ok ? t : start) * C;
        const size_t zrow = (size_t)(ok ? t : start) * H * D + (size_t)h * D;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = lane_elem<DS>(r, i);
            const bool in = ok && d < D;
            in_q[i] = in ? load_f32<TI>(x, row + (size_t)kh * D + d) : 0.f;
            in_k[i] = in ? load_f32<TI>(x, row + (size_t)(G + kh) * D + d) : 0.f;
            in_z[i] = in ? a.g[zrow + d] : 0.f;
        }
        const int j = col0 + r;
        in_v = (ok && j < Dv) ? load_f32<TI>(x, row + (size_t)2 * G * D + (size_t)h * Dv + j) : 0.f;
        in_b = (ok && r == 0) ? load_f32<TB>(bl, (size_t)t * a.ldb + h) : 0.f;
    };
    fetch(start);
    for (int t0 = start; t0 < end; t0 += TILE) {
        const int nt = min(TILE, end - t0);
        __syncthreads();        // the tile before has been read
        if (cl < TILE) {
            float sq = 0.f, sk = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                sq = fmaf(in_q[i], in_q[i], sq);
                sk = fmaf(in_k[i], in_k[i], sk);
            }
            sq = row16_sum(sq);
            sk = row16_sum(sk);
            const float rq = q_scale / sqrtf(sq + 1e-6f), rk = 1.0f / sqrtf(sk + 1e-6f);
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = lane_elem<DS>(r, i);
                qs[cl][d] = in_q[i] * rq;
                ks[cl][d] = in_k[i] * rk;
                gs[cl][d] = in_z[i];
            }
            vs[cl][r] = in_v;
            if (r == 0) beta_s[cl] = 1.0f / (1.0f + expf(-in_b));
        }
        __syncthreads();
        if (t0 + TILE < end) fetch(t0 + TILE);      // on its way while this tile is worked through
        auto token = [&](int tt) {
            float p = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = lane_elem<DS>(r, i);
                S[i] *= gs[tt][d];
                p = fmaf(ks[tt][d], S[i], p);
            }
            p = row16_sum(p);
            const float u = beta_s[tt] * (vs[tt][cl] - p);
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = lane_elem<DS>(r, i);
                S[i] = fmaf(ks[tt][d], u, S[i]);
                acc = fmaf(qs[tt][d], S[i], acc);
            }
            acc = row16_sum(acc);
            if (r == 0 && col < Dv) a.o[((size_t)(t0 + tt) * H + h) * Dv + col] = acc;
        };
        if (nt == TILE) {
#pragma unroll
            for (int tt = 0; tt < TILE; ++tt) token(tt);
        } else {
            for (int tt = 0; tt < nt; ++tt) token(tt);
        }
    }
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = lane_elem<DS>(r, i);
        if (col < Dv && d < D) S_head[(size_t)col * D + d] = S[i];
    }
}

extern "C" int vt_delta_rule_channel(const void* qkv, int dtype, const void* beta, int beta_dtype, long long ldb,
                                     const float* g, float* state, long long slot_stride,
                                     const int* entry_start, const int* slots, float* o, int n_entries, int H, int G, int D,
                                     int Dv, hipStream_t stream) {
    VT_REQUIRE(n_entries >= 0 && H > 0 && G > 0 && H % G == 0, "vt_delta_rule_channel: bad heads %d/%d", H, G);
    VT_REQUIRE(D > 0 && D <= 256 && Dv > 0, "vt_delta_rule_channel: head sizes %d/%d (keys up to 256)", D, Dv);
    VT_REQUIRE(slot_stride >= (long long)H * D * Dv, "vt_delta_rule_channel: state slots are too short");
    VT_REQUIRE(ldb >= H, "vt_delta_rule_channel: rows of write-strength logits are too short");
    VT_REQUIRE(H <= 65535, "vt_delta_rule_channel: too many heads (%d)", H);
    if (n_entries == 0) return 0;
    ChannelDeltaArgs a;
    a.qkv = qkv; a.beta = beta; a.g = g; a.state = state; a.entry_start = entry_start; a.slots = slots;
    a.o = o; a.slot_stride = slot_stride; a.ldb = ldb; a.H = H; a.G = G; a.D = D; a.Dv = Dv;
    const int share = (D + 15) / 16;
    const dim3 grid(n_entries, H, (Dv + DELTA_GROUPS - 1) / DELTA_GROUPS);
#define VT_CDELTA(TI, TB)                                                                                  \
    do {                                                                                                   \
        if (share <= 1) delta_rule_channel_kernel<TI, TB, 1, 16><<<grid, 256, 0, stream>>>(a);             \
        else if (share <= 2) delta_rule_channel_kernel<TI, TB, 2, 16><<<grid, 256, 0, stream>>>(a);        \
        else if (share <= 4) delta_rule_channel_kernel<TI, TB, 4, 16><<<grid, 256, 0, stream>>>(a);        \
        else if (share <= 8) delta_rule_channel_kernel<TI, TB, 8, 16><<<grid, 256, 0, stream>>>(a);        \
        else delta_rule_channel_kernel<TI, TB, 16, 16><<<grid, 256, 0, stream>>>(a);                       \
    } while (0)
    if (dtype == VT_F32 && beta_dtype == VT_F32) VT_CDELTA(float, float);
    else if (dtype == VT_BF16 && beta_dtype == VT_F32) VT_CDELTA(bf16_t, float);
    else if (dtype == VT_BF16 && beta_dtype == VT_BF16) VT_CDELTA(bf16_t, bf16_t);
    else return vt_fail("vt_delta_rule_channel: dtypes %d / %d are not handled", dtype, beta_dtype);
#undef VT_CDELTA
    VT_CHECK_LAUNCH("vt_delta_rule_channel");
    return 0;
}

// ---------------------------------------------------------------------------
struct MemoryArgs {
    const void* x;          // [n][ldx]: per head D queries from q_col, D keys from k_col, Dv values from v_col, and one
                            // logit per head of the input gate from i_col and of the forget gate from f_col
    const float* i_bias;    // [H] or null
    const float* f_bias;    // [H] or null
    float* state;           // slot s: state + s * slot_stride: [H][Dv][D] matrices, then [H][ZB][D] normalizers, then
                            // [H][ZB] maxima, ZB = blocks of 16 value columns
    const int* entry_start;
    const int* slots;
    float* o;               // [n][H][Dv]
    long long ldx, slot_stride;
    int q_col, k_col, v_col, i_col, f_col;
    int H, D, Dv;
    float cap, q_scale;
};

__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

template <typename TI, int DS, int TILE>
__global__ __launch_bounds__(256) void matrix_memory_kernel(MemoryArgs a) {
    constexpr int DP = 16 * DS;
    __shared__ __attribute__((aligned(16))) float qs[TILE][DP];
    __shared__ __attribute__((aligned(16))) float ks[TILE][DP];
    __shared__ float vs[TILE][DELTA_GROUPS];
    __shared__ float i_s[TILE], f_s[TILE], keep_s[TILE], put_s[TILE], floor_s[TILE];

    const int e = blockIdx.x, h = blockIdx.y, zb = blockIdx.z, col0 = zb * DELTA_GROUPS;
    const int ZB = gridDim.z;
    const int tid = threadIdx.x;
    const int r = tid & 15, cl = tid >> 4;
    const int D = a.D, Dv = a.Dv, H = a.H;
    const int start = a.entry_start[e], end = a.entry_start[e + 1];
    float* slot = a.state + (size_t)a.slots[e] * a.slot_stride;
    float* S_head = slot + (size_t)h * Dv * D;
    float* n_own = slot + (size_t)H * Dv * D + ((size_t)h * ZB + zb) * D;
    float* m_own = slot + (size_t)H * Dv * D + (size_t)H * ZB * D + (size_t)h * ZB + zb;
    const TI* x = (const TI*)a.x;
    const int col = col0 + cl;
    const float ib = a.i_bias ? a.i_bias[h] : 0.f, fb = a.f_bias ? a.f_bias[h] : 0.f;

    float S[DS], nn[DS];
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = lane_elem<DS>(r, i);
        S[i] = (col < Dv && d < D) ? S_head[(size_t)col * D + d] : 0.f;
        nn[i] = d < D ? n_own[d] : 0.f;
    }
    float m = *m_own;

    float in_q[DS], in_k[DS], in_v = 0.f, in_i = 0.f, in_f = 0.f;
    auto fetch = [&](int t0) {
        const int t = t0 + cl;
        const bool ok = cl < TILE && t < end;
        const size_t row = (size_t)(ok ? t : start) * a.ldx;
#pragma unroll
        for (int i = 0; i < DS; ++i) {
            const int d = lane_elem<DS>(r, i);
            const bool in = ok && d < D;
            in_q[i] = in ? load_f32<TI>(x, row + a.q_col + (size_t)h * D + d) : 0.f;
            in_k[i] = in ? load_f32<TI>(x, row + a.k_col + (size_t)h * D + d) : 0.f;
        }
        const int j = col0 + r;
        in_v = (ok && j < Dv) ? load_f32<TI>(x, row + a.v_col + (size_t)h * Dv + j) : 0.f;
        if (ok && r == 0) {
            in_i = load_f32<TI>(x, row + a.i_col + h);
            in_f = load_f32<TI>(x, row + a.f_col + h);
        }
    };
    fetch(start);
    for (int t0 = start; t0 < end; t0 += TILE) {
        const int nt = min(TILE, end - t0);
        __syncthreads();        // the tile before has been read
        if (cl < TILE) {
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = lane_elem<DS>(r, i);
                qs[cl][d] = in_q[i] * a.q_scale;
                ks[cl][d] = in_k[i];
            }
            vs[cl][r] = in_v;
            if (r == 0) {
                // the gates' logarithms, capped (cap 0: as they come)
                const float zi = in_i + ib, zf = in_f + fb;
                i_s[cl] = a.cap > 0.f ? a.cap * tanhf(zi / a.cap) : zi;
                f_s[cl] = log_sigmoid_f(a.cap > 0.f ? a.cap * tanhf(zf / a.cap) : zf);
            }
        }
        __syncthreads();
        if (t0 + TILE < end) fetch(t0 + TILE);      // on its way while this tile is worked through
        {
            // The running maximum is a chain of additions and maxima, token by token, that every thread walks for
            // itself (it is the same whatever the tile); the thread of token cl then works out that token's three
            // exponentials, so that they leave the recurrence below: keep = e^(f + m - m'), put = e^(i - m'), and
            // e^(-m'), the least that the normalizer's product counts as.
            float lf_own = 0.f, li_own = 0.f, m_own_new = 0.f;
#pragma unroll
            for (int tt = 0; tt < TILE; ++tt) {
                if (tt < nt) {
                    const float lf = f_s[tt] + m, li = i_s[tt];
                    m = fmaxf(lf, li);
                    if (tt == cl) { lf_own = lf; li_own = li; m_own_new = m; }
                }
            }
            if (cl < nt && r == 0) {
                keep_s[cl] = expf(lf_own - m_own_new);
                put_s[cl] = expf(li_own - m_own_new);
                floor_s[cl] = expf(-m_own_new);
            }
        }
        __syncthreads();
        auto token = [&](int tt) {
            const float keep = keep_s[tt], put = put_s[tt];
            const float pv = put * vs[tt][cl];
            float acc = 0.f, den = 0.f;
#pragma unroll
            for (int i = 0; i < DS; ++i) {
                const int d = lane_elem<DS>(r, i);
                const float kd = ks[tt][d], qd = qs[tt][d];
                S[i] = fmaf(keep, S[i], kd * pv);
                nn[i] = fmaf(keep, nn[i], kd * put);
                acc = fmaf(qd, S[i], acc);
                den = fmaf(qd, nn[i], den);
            }
            acc = row16_sum(acc);
            den = row16_sum(den);
            if (r == 0 && col < Dv)
                a.o[((size_t)(t0 + tt) * H + h) * Dv + col] = acc / (fmaxf(fabsf(den), floor_s[tt]) + 1e-6f);
        };
        if (nt == TILE) {
#pragma unroll
            for (int tt = 0; tt < TILE; ++tt) token(tt);
        } else {
            for (int tt = 0; tt < nt; ++tt) token(tt);
        }
    }
#pragma unroll
    for (int i = 0; i < DS; ++i) {
        const int d = lane_elem<DS>(r, i);
        if (col < Dv && d < D) S_head[(size_t)col * D + d] = S[i];
        if (cl == 0 && d < D) n_own[d] = nn[i];
    }
    if (tid == 0) *m_own = m;
}

extern "C" long long vt_matrix_memory_state_floats(int H, int D, int Dv) {
    const long long zb = (Dv + DELTA_GROUPS - 1) / DELTA_GROUPS;
    return (long long)H * Dv * D + (long long)H * zb * D + (long long)H * zb;
}

extern "C" int vt_matrix_memory(const void* x, int dtype, long long ldx, int q_col, int k_col, int v_col, int i_col, int f_col,
                                const float* i_bias, const float* f_bias, float* state, long long slot_stride,
                                const int* entry_start, const int* slots, float* o, int n_entries, int H, int D, int Dv,
                                float cap, float q_scale, hipStream_t stream) {
    VT_REQUIRE(n_entries >= 0 && H > 0 && H <= 65535, "vt_matrix_memory: bad heads %d", H);
    VT_REQUIRE(D > 0 && D <= 256 && Dv > 0, "vt_matrix_memory: head sizes %d/%d (keys up to 256)", D, Dv);
    VT_REQUIRE(slot_stride >= vt_matrix_memory_state_floats(H, D, Dv), "vt_matrix_memory: state slots are too short");
    VT_REQUIRE(min(min(q_col, k_col), min(v_col, min(i_col, f_col))) >= 0 && ldx >= max(q_col, k_col) + (long long)H * D &&
               ldx >= v_col + (long long)H * Dv && ldx >= max(i_col, f_col) + (long long)H,
               "vt_matrix_memory: rows are too short for their columns");
    VT_REQUIRE(cap >= 0.f, "vt_matrix_memory: a negative cap");
    if (n_entries == 0) return 0;
    MemoryArgs a;
    a.x = x; a.i_bias = i_bias; a.f_bias = f_bias; a.state = state; a.entry_start = entry_start; a.slots = slots; a.o = o;
    a.ldx = ldx; a.slot_stride = slot_stride; a.q_col = q_col; a.k_col = k_col; a.v_col = v_col; a.i_col = i_col; a.f_col = f_col;
    a.H = H; a.D = D; a.Dv = Dv; a.cap = cap; a.q_scale = q_scale;
    const int share = (D + 15) / 16;
    const dim3 grid(n_entries, H, (Dv + DELTA_GROUPS - 1) / DELTA_GROUPS);
#define VT_MEMORY(TI)                                                                              \
    do {                                                                                           \
        if (share <= 1) matrix_memory_kernel<TI, 1, 16><<<grid, 256, 0, stream>>>(a);              \
        else if (share <= 2) matrix_memory_kernel<TI, 2, 16><<<grid, 256, 0, stream>>>(a);         \
        else if (share <= 4) matrix_memory_kernel<TI, 4, 16><<<grid, 256, 0, stream>>>(a);         \
        else if (share <= 8) matrix_memory_kernel<TI, 8, 16><<<grid, 256, 0, stream>>>(a);         \
        else matrix_memory_kernel<TI, 16, 16><<<grid, 256, 0, stream>>>(a);                        \
    } while (0)
    if (dtype == VT_F32) VT_MEMORY(float);
    else if (dtype == VT_BF16) VT_MEMORY(bf16_t);
    else return vt_fail("vt_matrix_memory: unknown dtype %d", dtype);
#undef VT_MEMORY
    VT_CHECK_LAUNCH("vt_matrix_memory");
    return 0;
}
