// The 16-bit attention of vt_attn_masked.hip on the matrix cores, for steps that bring portions of prompts: capped
// scores, chunk or window masks, key and value heads of different sizes (both multiples of 16, fixed when this file
// is compiled: VT_KEY_DIM, VT_VALUE_DIM), one gate per head.
//
// A wave takes a tile of up to 16 consecutive tokens of one request and one query head; the host lists the tiles
// (first row, rows).  A turn of the loop takes 32 keys, asked for a turn ahead.  Per 16 keys (one page, or part of one:
// pages hold a multiple of 16 keys):
//     S^T = K Q^T      [16 keys x 16 queries], v_mfma_f32_16x16x16 over the key size; A = K rows from the page
//                      ([kv head][slot][D]: a lane reads 4 consecutive elements of its key), B = Q from registers
//     cap, mask, running maximum and sum per query (a query is a column: its 16 scores lie in 4 lanes x 4 registers)
//     O^T += V^T P^T   [Dv x 16 queries]; A = V^T from the page ([kv head][Dv][slot]: a lane reads 4 consecutive keys of
//                      its value element), B = P^T, which is exactly what the lane holds of S^T
// so the probabilities never leave the registers.  Scores, softmax and sums are float32.
// With `slopes`, slopes[head] * (position - key index) is taken off every score; with `sink`, exp(sink[head]) joins
// the softmax's denominator (a key that holds no value).  Further forms, each switched on by its pointer or flag:
// `dist_r1`, `dist_r2`: r1[head] * ln(1 + r2[head] * (position - key index)) is taken off every score (base 2:
// r1 * log2(1 + r2 d), the hardware's logarithm); `score_shift`: a number per head added to every score;
// sigmoid_weights: the weight of a seen key is sigmoid(score) = 1 / (1 + 2^-score'), nothing is normalized;
// gate_wide: one gate logit per output element, gate[token][head * Dv + d], instead of one per head.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

#ifndef VT_KEY_DIM
#error "compile with -DVT_KEY_DIM=<multiple of 16> -DVT_VALUE_DIM=<multiple of 16>"
#endif
static_assert(VT_KEY_DIM % 16 == 0 && VT_KEY_DIM >= 16 && VT_KEY_DIM <= 256, "key size");
static_assert(VT_VALUE_DIM % 16 == 0 && VT_VALUE_DIM >= 16 && VT_VALUE_DIM <= 256, "value size");

typedef __attribute__((ext_vector_type(4))) float f32x4;

struct MfmaArgs {
    const bf16_t* q;        // [n][H][D]
    const bf16_t* k_pages;  // [page][G][slot][D]
    const bf16_t* v_pages;  // [page][G][Dv][slot]
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    const int* tiles;       // [n_tiles][2]: first row, rows (1..16), all of one request
    const void* gate;       // gate[t * ldg + h], or null
    const float* sink;      // [H] or null
    const float* slopes;    // [H] or null
    const float* dist_r1;   // [H] each, or null
    const float* dist_r2;
    const float* score_shift;   // [H] or null
    bf16_t* out;            // [n][H][Dv]
    long long ldg;
    int n_tiles, H, G, page_size, max_blocks, num_pages, window, chunk, gate_f32, sigmoid_weights, gate_wide;
    float scale, cap;
};

// what the score's optional forms take off or add, in the base-2 domain: key j seen from position pos
struct ScoreForms {
    float slope2, r1, r2, shift2;
    bool has_slope, has_log;
    __device__ __forceinline__ float apply(float sc, int pos, int j) const {
        const float dist = (float)max(pos - j, 0);
        if (has_slope) sc -= slope2 * dist;
        if (has_log) sc -= r1 * __builtin_amdgcn_logf(fmaf(r2, dist, 1.0f));
        return sc + shift2;
    }
};
__device__ __forceinline__ ScoreForms score_forms(const float* slopes, const float* r1, const float* r2, const float* shift, int h) {
    const float LOG2E = 1.4426950408889634f;
    ScoreForms f;
    f.has_slope = slopes != nullptr;
    f.has_log = r1 != nullptr;
    f.slope2 = slopes ? slopes[h] * LOG2E : 0.f;
    f.r1 = r1 ? r1[h] : 0.f;          // r1 ln(x) log2(e) = r1 log2(x)
    f.r2 = r1 ? r2[h] : 0.f;
    f.shift2 = shift ? shift[h] * LOG2E : 0.f;
    return f;
}
// the gate on output element d of head h of token t
__device__ __forceinline__ float gate_at(const void* gate, int gate_f32, long long ldg, int t, size_t column) {
    const size_t gi = (size_t)t * ldg + column;
    const float z = gate_f32 ? ((const float*)gate)[gi] : bf16_to_f32(((const bf16_t*)gate)[gi]);
    return 1.0f / (1.0f + expf(-z));
}

__device__ __forceinline__ vt_lowp4_t load4(const bf16_t* p) { return *(const vt_lowp4_t*)p; }

__global__ __launch_bounds__(256) void attn_masked_mfma_kernel(MfmaArgs a) {
    constexpr int D = VT_KEY_DIM, DV = VT_VALUE_DIM, NK = D / 16, NV = DV / 16;
    const int lane = threadIdx.x & 63;
    const int item = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (item >= a.n_tiles * a.H) return;
    const int tile = item / a.H, h = item % a.H;
    const int kvh = h / (a.H / a.G);
    const int first = a.tiles[2 * tile], rows = a.tiles[2 * tile + 1];
    const int r = lane & 15, grp = lane >> 4;
    const bool row_ok = r < rows;
    const int t = first + (row_ok ? r : 0);
    const int pos = a.positions[t];
    const int pos_first = a.positions[first], pos_last = a.positions[first + rows - 1];
    const int* bt = a.block_table + (size_t)a.tok_entry[first] * a.max_blocks;
    const int ps = a.page_size;

    int lo_r = a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo_r = max(lo_r, pos - a.window + 1);
    int lo = a.chunk > 0 ? (pos_first / a.chunk) * a.chunk : 0;       // the first row's bound is the lowest
    if (a.window > 0) lo = max(lo, pos_first - a.window + 1);

    vt_lowp4_t qf[NK];
    {
        const bf16_t* qr = a.q + ((size_t)t * a.H + h) * D + grp * 4;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
            qf[kk] = load4(qr + kk * 16);
            if (!row_ok) qf[kk] = (vt_lowp4_t){0, 0, 0, 0};
        }
    }
    f32x4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const float nan = __int_as_float(0x7fc00000);

    // Scores are kept times log2(e), so that every exponential is the hardware's 2^x.  The cap, with y = scale s / cap:
    // cap tanh(y) = cap (1 - 2 / (1 + e^(2y))), e^(2y) = 2^(s c1).
    const float LOG2E = 1.4426950408889634f;
    const float c1 = a.cap > 0.f ? a.scale * 2.0f * LOG2E / a.cap : a.scale * LOG2E;
    const float c2 = a.cap * LOG2E;
    const ScoreForms forms = score_forms(a.slopes, a.dist_r1, a.dist_r2, a.score_shift, h);
    const bool forms_on = a.slopes || a.dist_r1 || a.score_shift;
    const bool sig = a.sigmoid_weights != 0;
    const int lo_last = [&] {
        int v = a.chunk > 0 ? (pos_last / a.chunk) * a.chunk : 0;
        if (a.window > 0) v = max(v, pos_last - a.window + 1);
        return v;
    }();

    // 32 keys a turn, as two runs of 16 (each inside one page).  A turn's keys and values are asked for a turn ahead,
    // and the pages they lie in two turns ahead, so that no turn waits for a page number before it can ask for keys.
    vt_lowp4_t kf[2][NK], vf[2][NV], kn[2][NK], vn[2][NV];
    bool ok_now[2] = {false, false}, ok_next[2] = {false, false};
    auto page_of = [&](int kt) -> int {
        const int blk = kt / ps;
        return blk < a.max_blocks ? bt[blk] : -1;
    };
    auto fetch = [&](int kt, int pg, vt_lowp4_t* kd, vt_lowp4_t* vd, bool& ok) {
        ok = pg >= 0 && pg < a.num_pages;
        pg = ok ? pg : 0;
        const int slot0 = kt % ps;
        const bf16_t* kp = a.k_pages + (((size_t)pg * a.G + kvh) * ps + slot0 + r) * D + grp * 4;
        const bf16_t* vp = a.v_pages + (((size_t)pg * a.G + kvh) * DV + r) * ps + slot0 + grp * 4;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) kd[kk] = load4(kp + kk * 16);
#pragma unroll
        for (int v = 0; v < NV; ++v) vd[v] = load4(vp + (size_t)v * 16 * ps);
    };
    const int kt0 = (lo / 16) * 16;
    fetch(kt0, page_of(kt0), kn[0], vn[0], ok_next[0]);
    fetch(kt0 + 16, page_of(kt0 + 16), kn[1], vn[1], ok_next[1]);
    int pg_a = page_of(kt0 + 32), pg_b = page_of(kt0 + 48);
    for (int kt = kt0; kt <= pos_last; kt += 32) {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) kf[u][kk] = kn[u][kk];
#pragma unroll
            for (int v = 0; v < NV; ++v) vf[u][v] = vn[u][v];
            ok_now[u] = ok_next[u];
        }
        if (kt + 32 <= pos_last) {
            fetch(kt + 32, pg_a, kn[0], vn[0], ok_next[0]);
            fetch(kt + 48, pg_b, kn[1], vn[1], ok_next[1]);
            pg_a = page_of(kt + 64);
            pg_b = page_of(kt + 80);
        }
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
            s0 = VT_MFMA_16X16X16(kf[0][kk], qf[kk], s0);
            s1 = VT_MFMA_16X16X16(kf[1][kk], qf[kk], s1);
        }
        float sc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float x = (i < 4 ? s0[i] : s1[i - 4]) * c1;
            if (a.cap > 0.f) {
                const float e = __builtin_amdgcn_exp2f(x);
                sc[i] = fmaf(-2.0f * c2, __builtin_amdgcn_rcpf(1.0f + e), c2);
            } else {
                sc[i] = x;
            }
        }
        if (forms_on) {
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[i] = forms.apply(sc[i], pos, kt + (i < 4 ? 0 : 16) + grp * 4 + (i & 3));
        }
        // a turn that every row sees whole needs no mask
        const bool whole = kt + 31 <= pos_first && kt >= lo_last && ok_now[0] && ok_now[1];
        if (!whole) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int j = kt + (i < 4 ? 0 : 16) + grp * 4 + (i & 3);
                const bool seen = row_ok && j <= pos && j >= lo_r;
                // (a missing page must show, not pass as a masked key)
                sc[i] = seen ? (ok_now[i >> 2] ? sc[i] : nan) : -INFINITY;
            }
        }
        float p[8], alpha = 1.f;
        if (sig) {
            // every key's weight stands alone: 1 / (1 + 2^-s), and 0 for a masked key (s = -inf)
#pragma unroll
            for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-sc[i]));
        } else {
            float mt = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
            mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float m_new = fmaxf(m, mt);
            const float mref = (m_new == -INFINITY) ? 0.f : m_new;
            alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p[i] = __builtin_amdgcn_exp2f(sc[i] - mref);
                psum += p[i];
            }
            l = l * alpha + psum;
            m = m_new;
        }
        struct U2 { unsigned a, b; };
        const U2 pk0 = {vt_pack2(p[0], p[1]), vt_pack2(p[2], p[3])}, pk1 = {vt_pack2(p[4], p[5]), vt_pack2(p[6], p[7])};
        const vt_lowp4_t pf0 = __builtin_bit_cast(vt_lowp4_t, pk0), pf1 = __builtin_bit_cast(vt_lowp4_t, pk1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            acc[v] *= alpha;
            acc[v] = VT_MFMA_16X16X16(vf[0][v], pf0, acc[v]);
            acc[v] = VT_MFMA_16X16X16(vf[1][v], pf1, acc[v]);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    if (a.sink && !sig) {
        // the sink is one more score with no value behind it (scores are kept times log2 e)
        const float sk = a.sink[h] * LOG2E;
        const float m_all = fmaxf(m, sk);
        const float keep = __builtin_amdgcn_exp2f(m - m_all);
        l = l * keep + __builtin_amdgcn_exp2f(sk - m_all);
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[v] *= keep;
    }
    if (sig) l = 1.f;
    const float f = ((a.gate && !a.gate_wide) ? gate_at(a.gate, a.gate_f32, a.ldg, t, h) : 1.f) / l;
    bf16_t* o = a.out + ((size_t)t * a.H + h) * DV + grp * 4;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float g4[4] = {f, f, f, f};
        if (a.gate && a.gate_wide) {
#pragma unroll
            for (int i = 0; i < 4; ++i) g4[i] = f * gate_at(a.gate, a.gate_f32, a.ldg, t, (size_t)h * DV + v * 16 + grp * 4 + i);
        }
        struct { unsigned a, b; } ok = {vt_pack2(acc[v][0] * g4[0], acc[v][1] * g4[1]), vt_pack2(acc[v][2] * g4[2], acc[v][3] * g4[3])};
        *(uint2*)(o + v * 16) = __builtin_bit_cast(uint2, ok);
    }
}

// The same work with the block's four waves sharing what they read: when a key/value head serves a multiple of four
// query heads, the four waves of a block are four heads of one group on the same 16 tokens, so they want the same keys
// and values.  The block brings a turn's 32 keys and their values from the pages once (every thread a few 16-byte
// pieces, a turn ahead, into registers), puts them into LDS (two buffers, rows padded against bank conflicts: one
// barrier a turn), and every wave reads its matrix operands from there.
__global__ __launch_bounds__(256) void attn_masked_mfma_shared_kernel(MfmaArgs a) {
    constexpr int D = VT_KEY_DIM, DV = VT_VALUE_DIM, NV = DV / 16;
    constexpr int NK32 = D / 32;                // products of 32 key elements; a key size that is no multiple of 32 ends in one of 16
    constexpr bool TAIL = D % 32 != 0;
    constexpr int KROW = D + 8;                 // elements of a key's row in LDS (rows stay 16-byte aligned)
    constexpr int VROW = 32 + 4;                // elements of a value element's row in LDS: 32 keys
    constexpr int KP = (4 * D + 255) / 256;     // 16-byte pieces of a turn's keys per thread
    constexpr int VP = (4 * DV + 255) / 256;    // ... of its values
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][32 * KROW];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][DV * VROW];

    const int tid = threadIdx.x, lane = tid & 63;
    const int item = blockIdx.x * 4 + (tid >> 6);       // (the launch has whole blocks: the heads are a multiple of four)
    const int tile = item / a.H, h = item % a.H;
    const int kvh = h / (a.H / a.G);
    const int first = a.tiles[2 * tile], rows = a.tiles[2 * tile + 1];
    const int r = lane & 15, grp = lane >> 4;
    const bool row_ok = r < rows;
    const int t = first + (row_ok ? r : 0);
    const int pos = a.positions[t];
    const int pos_first = a.positions[first], pos_last = a.positions[first + rows - 1];
    const int* bt = a.block_table + (size_t)a.tok_entry[first] * a.max_blocks;
    const int ps = a.page_size;

    int lo_r = a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo_r = max(lo_r, pos - a.window + 1);
    int lo = a.chunk > 0 ? (pos_first / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo = max(lo, pos_first - a.window + 1);
    int lo_last = a.chunk > 0 ? (pos_last / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo_last = max(lo_last, pos_last - a.window + 1);

    // queries as the second operand of v_mfma_f32_16x16x32: a lane holds 8 consecutive elements of its row
    // (a key size that is no multiple of 32 ends in 16 elements: they take the same instruction with four elements
    // and four zeros per lane, so that one kind of product feeds an accumulator)
    vt_lowp8_t qf[NK32 > 0 ? NK32 : 1];
    auto low_half = [](const bf16_t* p) -> vt_lowp8_t {             // four elements from p, then four zeros
        const uint2 v = *(const uint2*)p;
        return __builtin_bit_cast(vt_lowp8_t, make_uint4(v.x, v.y, 0u, 0u));
    };
    vt_lowp8_t qtail = __builtin_bit_cast(vt_lowp8_t, make_uint4(0u, 0u, 0u, 0u));
    {
        const bf16_t* qrow = a.q + ((size_t)t * a.H + h) * D;
        const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int kk = 0; kk < NK32; ++kk) {
            const uint4 raw = row_ok ? *(const uint4*)(qrow + kk * 32 + grp * 8) : zero4;
            qf[kk] = __builtin_bit_cast(vt_lowp8_t, raw);
        }
        if (TAIL && row_ok) qtail = low_half(qrow + (D - 16) + grp * 4);
    }
    f32x4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const float nan = __int_as_float(0x7fc00000);
    const float LOG2E = 1.4426950408889634f;
    const float c1 = a.cap > 0.f ? a.scale * 2.0f * LOG2E / a.cap : a.scale * LOG2E;
    const float c2 = a.cap * LOG2E;
    const ScoreForms forms = score_forms(a.slopes, a.dist_r1, a.dist_r2, a.score_shift, h);
    const bool forms_on = a.slopes || a.dist_r1 || a.score_shift;
    const bool sig = a.sigmoid_weights != 0;

    auto page_of = [&](int kt) -> int {
        const int blk = kt / ps;
        return blk < a.max_blocks ? bt[blk] : -1;
    };
    uint4 kreg[KP], vreg[VP];
    bool ok_next[2] = {false, false}, ok_now[2] = {false, false};
    auto fetch = [&](int kt, int pg0, int pg1) {
        ok_next[0] = pg0 >= 0 && pg0 < a.num_pages;
        ok_next[1] = pg1 >= 0 && pg1 < a.num_pages;
        const size_t base0 = ((size_t)(ok_next[0] ? pg0 : 0) * a.G + kvh), base1 = ((size_t)(ok_next[1] ? pg1 : 0) * a.G + kvh);
        const int slot_a = kt % ps, slot_b = (kt + 16) % ps;
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int p = tid + 256 * i;
            if (p < 4 * D) {
                const int key = p / (D / 8), off = (p % (D / 8)) * 8;
                const bf16_t* src = a.k_pages + ((key < 16 ? base0 : base1) * ps + (key < 16 ? slot_a + key : slot_b + key - 16)) * D + off;
                kreg[i] = *(const uint4*)src;
            }
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int p = tid + 256 * i;
            if (p < 4 * DV) {
                const int row = p >> 2, q4 = p & 3;
                const bf16_t* src = a.v_pages + ((q4 < 2 ? base0 : base1) * DV + row) * ps + (q4 < 2 ? slot_a : slot_b) + (q4 & 1) * 8;
                vreg[i] = *(const uint4*)src;
            }
        }
    };
    auto to_lds = [&](int b) {
#pragma unroll
        for (int i = 0; i < KP; ++i) {
            const int p = tid + 256 * i;
            if (p < 4 * D) {
                const int key = p / (D / 8), off = (p % (D / 8)) * 8;
                uint2* dst = (uint2*)&k_lds[b][key * KROW + off];
                dst[0] = make_uint2(kreg[i].x, kreg[i].y);
                dst[1] = make_uint2(kreg[i].z, kreg[i].w);
            }
        }
#pragma unroll
        for (int i = 0; i < VP; ++i) {
            const int p = tid + 256 * i;
            if (p < 4 * DV) {
                const int row = p >> 2, q4 = p & 3;
                uint2* dst = (uint2*)&v_lds[b][row * VROW + q4 * 8];
                dst[0] = make_uint2(vreg[i].x, vreg[i].y);
                dst[1] = make_uint2(vreg[i].z, vreg[i].w);
            }
        }
    };

    const int kt0 = (lo / 16) * 16;
    fetch(kt0, page_of(kt0), page_of(kt0 + 16));
    int pg_a = page_of(kt0 + 32), pg_b = page_of(kt0 + 48);
    int b = 0;
    for (int kt = kt0; kt <= pos_last; kt += 32) {
        to_lds(b);
        ok_now[0] = ok_next[0];
        ok_now[1] = ok_next[1];
        if (kt + 32 <= pos_last) {
            fetch(kt + 32, pg_a, pg_b);
            pg_a = page_of(kt + 64);
            pg_b = page_of(kt + 80);
        }
        __syncthreads();
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
        const bf16_t* kl = &k_lds[b][r * KROW];
#pragma unroll
        for (int kk = 0; kk < NK32; ++kk) {
            const vt_lowp8_t k0 = __builtin_bit_cast(vt_lowp8_t, *(const uint4*)(kl + kk * 32 + grp * 8));
            const vt_lowp8_t k1 = __builtin_bit_cast(vt_lowp8_t, *(const uint4*)(kl + 16 * KROW + kk * 32 + grp * 8));
            s0 = VT_MFMA_16X16X32(k0, qf[kk], s0);
            s1 = VT_MFMA_16X16X32(k1, qf[kk], s1);
        }
        if (TAIL) {
            s0 = VT_MFMA_16X16X32(low_half(kl + (D - 16) + grp * 4), qtail, s0);
            s1 = VT_MFMA_16X16X32(low_half(kl + 16 * KROW + (D - 16) + grp * 4), qtail, s1);
        }
        float sc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float x = (i < 4 ? s0[i] : s1[i - 4]) * c1;
            if (a.cap > 0.f) {
                const float e = __builtin_amdgcn_exp2f(x);
                sc[i] = fmaf(-2.0f * c2, __builtin_amdgcn_rcpf(1.0f + e), c2);
            } else {
                sc[i] = x;
            }
        }
        if (forms_on) {
#pragma unroll
            for (int i = 0; i < 8; ++i) sc[i] = forms.apply(sc[i], pos, kt + (i < 4 ? 0 : 16) + grp * 4 + (i & 3));
        }
        const bool whole = kt + 31 <= pos_first && kt >= lo_last && ok_now[0] && ok_now[1];
        if (!whole) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int j = kt + (i < 4 ? 0 : 16) + grp * 4 + (i & 3);
                const bool seen = row_ok && j <= pos && j >= lo_r;
                sc[i] = seen ? (ok_now[i >> 2] ? sc[i] : nan) : -INFINITY;
            }
        }
        float p[8], alpha = 1.f;
        if (sig) {
            // every key's weight stands alone: 1 / (1 + 2^-s), and 0 for a masked key (s = -inf)
#pragma unroll
            for (int i = 0; i < 8; ++i) p[i] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-sc[i]));
        } else {
            float mt = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
            mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float m_new = fmaxf(m, mt);
            const float mref = (m_new == -INFINITY) ? 0.f : m_new;
            alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                p[i] = __builtin_amdgcn_exp2f(sc[i] - mref);
                psum += p[i];
            }
            l = l * alpha + psum;
            m = m_new;
        }
        // One product over the turn's 32 keys.  Its key index 8 grp + j stands for key 4 grp + j of the first run
        // (j < 4) and key 16 + 4 grp + j - 4 of the second: that is the order of the lane's eight probabilities, and the
        // values are read from LDS in the same order.
        const uint4 praw = make_uint4(vt_pack2(p[0], p[1]), vt_pack2(p[2], p[3]), vt_pack2(p[4], p[5]), vt_pack2(p[6], p[7]));
        const vt_lowp8_t pf = __builtin_bit_cast(vt_lowp8_t, praw);
        const bf16_t* vl = &v_lds[b][r * VROW + grp * 4];
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            const uint2 va = *(const uint2*)(vl + v * 16 * VROW), vb = *(const uint2*)(vl + v * 16 * VROW + 16);
            const vt_lowp8_t vf = __builtin_bit_cast(vt_lowp8_t, make_uint4(va.x, va.y, vb.x, vb.y));
            acc[v] *= alpha;
            acc[v] = VT_MFMA_16X16X32(vf, pf, acc[v]);
        }
        b ^= 1;
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    if (a.sink && !sig) {
        // the sink is one more score with no value behind it (scores are kept times log2 e)
        const float sk = a.sink[h] * LOG2E;
        const float m_all = fmaxf(m, sk);
        const float keep = __builtin_amdgcn_exp2f(m - m_all);
        l = l * keep + __builtin_amdgcn_exp2f(sk - m_all);
#pragma unroll
        for (int v = 0; v < NV; ++v) acc[v] *= keep;
    }
    if (sig) l = 1.f;
    const float f = ((a.gate && !a.gate_wide) ? gate_at(a.gate, a.gate_f32, a.ldg, t, h) : 1.f) / l;
    bf16_t* o = a.out + ((size_t)t * a.H + h) * DV + grp * 4;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        float g4[4] = {f, f, f, f};
        if (a.gate && a.gate_wide) {
#pragma unroll
            for (int i = 0; i < 4; ++i) g4[i] = f * gate_at(a.gate, a.gate_f32, a.ldg, t, (size_t)h * DV + v * 16 + grp * 4 + i);
        }
        struct { unsigned a, b; } ok = {vt_pack2(acc[v][0] * g4[0], acc[v][1] * g4[1]), vt_pack2(acc[v][2] * g4[2], acc[v][3] * g4[3])};
        *(uint2*)(o + v * 16) = __builtin_bit_cast(uint2, ok);
    }
}

// ---------------------------------------------------------------------------
// Steps of single tokens (decoding).  The 16 rows of the matrix products are not tokens but the query heads that share
// a key/value head, all of one token: one read of a key serves the whole group, which for a mixer whose heads all read
// one cache is every head.  The keys of a token are dealt out in turns of 32 to P = 4 x splits waves (turn i to wave
// i mod P), each wave keeps its own running maximum, sum and weighted values and leaves them in `part`; a second
// launch merges the P parts of every head, adds the sink to the denominator, applies the gate and writes the output.
// The grid depends on the number of tokens and on `splits` alone, the keys' range is read from device memory: a step
// can be recorded once and replayed.
//   part: [token][group tile][P][16 rows][DV + 4] floats: weighted values, then maximum and sum (base 2)
// ---------------------------------------------------------------------------
struct DecodeArgs {
    const bf16_t* q;        // [n][H][D]
    const bf16_t* k_pages;
    const bf16_t* v_pages;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    const float* sink;
    const float* slopes;
    const float* dist_r1;
    const float* dist_r2;
    const float* score_shift;
    const void* gate;
    float* part;
    bf16_t* out;            // [n][H][DV]
    long long ldg;
    int n, H, G, HT, P, page_size, max_blocks, num_pages, window, chunk, gate_f32, sigmoid_weights, gate_wide;
    float scale, cap;
};
#define DEC_ROW (VT_VALUE_DIM + 4)

__global__ __launch_bounds__(256) void attn_masked_decode_kernel(DecodeArgs a) {
    constexpr int D = VT_KEY_DIM, DV = VT_VALUE_DIM, NK = D / 16, NV = DV / 16;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r = lane & 15, grp = lane >> 4;
    const int p = blockIdx.x * 4 + wave, tile = blockIdx.y, t = blockIdx.z;
    const int group = a.H / a.G;
    const int kvh = tile / a.HT, ht = tile % a.HT;
    const int rows = min(16, group - ht * 16);
    const bool row_ok = r < rows;
    const int h = kvh * group + ht * 16 + (row_ok ? r : 0);
    const int pos = a.positions[t];
    const int* bt = a.block_table + (size_t)a.tok_entry[t] * a.max_blocks;
    const int ps = a.page_size;
    int lo = a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo = max(lo, pos - a.window + 1);
    const int kt0 = (lo / 16) * 16;
    const int turns = (pos - kt0) / 32 + 1;

    vt_lowp4_t qf[NK];
    {
        const bf16_t* qr = a.q + ((size_t)t * a.H + h) * D + grp * 4;
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
            qf[kk] = load4(qr + kk * 16);
            if (!row_ok) qf[kk] = (vt_lowp4_t){0, 0, 0, 0};
        }
    }
    f32x4 acc[NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) acc[v] = (f32x4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;
    const float nan = __int_as_float(0x7fc00000);
    const float LOG2E = 1.4426950408889634f;
    const float c1 = a.cap > 0.f ? a.scale * 2.0f * LOG2E / a.cap : a.scale * LOG2E;
    const float c2 = a.cap * LOG2E;
    const ScoreForms forms = score_forms(a.slopes, a.dist_r1, a.dist_r2, a.score_shift, h);
    const bool forms_on = a.slopes || a.dist_r1 || a.score_shift;
    const bool sig = a.sigmoid_weights != 0;

    for (int turn = p; turn < turns; turn += a.P) {
        const int kt = kt0 + turn * 32;
        vt_lowp4_t kf[2][NK], vf[2][NV];
        bool ok[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k0 = kt + 16 * u;
            const int blk = k0 / ps;
            int pg = blk < a.max_blocks ? bt[blk] : -1;
            ok[u] = pg >= 0 && pg < a.num_pages;
            pg = ok[u] ? pg : 0;
            const int slot0 = k0 % ps;
            const bf16_t* kp = a.k_pages + (((size_t)pg * a.G + kvh) * ps + slot0 + r) * D + grp * 4;
            const bf16_t* vp = a.v_pages + (((size_t)pg * a.G + kvh) * DV + r) * ps + slot0 + grp * 4;
#pragma unroll
            for (int kk = 0; kk < NK; ++kk) kf[u][kk] = load4(kp + kk * 16);
#pragma unroll
            for (int v = 0; v < NV; ++v) vf[u][v] = load4(vp + (size_t)v * 16 * ps);
        }
        f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
            s0 = VT_MFMA_16X16X16(kf[0][kk], qf[kk], s0);
            s1 = VT_MFMA_16X16X16(kf[1][kk], qf[kk], s1);
        }
        float sc[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float x = (i < 4 ? s0[i] : s1[i - 4]) * c1;
            if (a.cap > 0.f) {
                const float e = __builtin_amdgcn_exp2f(x);
                sc[i] = fmaf(-2.0f * c2, __builtin_amdgcn_rcpf(1.0f + e), c2);
            } else {
                sc[i] = x;
            }
            const int j = kt + (i < 4 ? 0 : 16) + grp * 4 + (i & 3);
            if (forms_on) sc[i] = forms.apply(sc[i], pos, j);
            const bool seen = row_ok && j <= pos && j >= lo;
            // (a missing page must show, not pass as a masked key)
            sc[i] = seen ? (ok[i >> 2] ? sc[i] : nan) : -INFINITY;
        }
        float pr[8], alpha = 1.f;
        if (sig) {
            // weights that stand alone: the part's "maximum" is 0 so that the merge adds the parts as they are
#pragma unroll
            for (int i = 0; i < 8; ++i) pr[i] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-sc[i]));
            m = 0.f;
        } else {
            float mt = fmaxf(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])), fmaxf(fmaxf(sc[4], sc[5]), fmaxf(sc[6], sc[7])));
            mt = fmaxf(mt, __shfl_xor(mt, 16, 64));
            mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float m_new = fmaxf(m, mt);
            const float mref = (m_new == -INFINITY) ? 0.f : m_new;
            alpha = (m == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m - m_new);
            float psum = 0.f;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                pr[i] = __builtin_amdgcn_exp2f(sc[i] - mref);
                psum += pr[i];
            }
            l = l * alpha + psum;
            m = m_new;
        }
        struct U2 { unsigned a, b; };
        const U2 pk0 = {vt_pack2(pr[0], pr[1]), vt_pack2(pr[2], pr[3])}, pk1 = {vt_pack2(pr[4], pr[5]), vt_pack2(pr[6], pr[7])};
        const vt_lowp4_t pf0 = __builtin_bit_cast(vt_lowp4_t, pk0), pf1 = __builtin_bit_cast(vt_lowp4_t, pk1);
#pragma unroll
        for (int v = 0; v < NV; ++v) {
            acc[v] *= alpha;
            acc[v] = VT_MFMA_16X16X16(vf[0][v], pf0, acc[v]);
            acc[v] = VT_MFMA_16X16X16(vf[1][v], pf1, acc[v]);
        }
    }
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!row_ok) return;
    float* dst = a.part + ((((size_t)t * a.G * a.HT + tile) * a.P + p) * 16 + r) * DEC_ROW;
#pragma unroll
    for (int v = 0; v < NV; ++v) *(float4*)(dst + v * 16 + grp * 4) = make_float4(acc[v][0], acc[v][1], acc[v][2], acc[v][3]);
    if (grp == 0) {
        dst[DV] = m;
        dst[DV + 1] = l;
    }
}

// A block per (token, head), a wave per 64 value elements: lane p takes part p's maximum and sum (P <= 64), the wave
// finds the common maximum and every part's weight 2^(m_p - m), and each lane then adds up its value element over the
// parts with those weights
// (from LDS; an empty part weighs nothing), loads that do not wait for one another.
#define MERGE_WAVES ((VT_VALUE_DIM + 63) / 64)
__global__ __launch_bounds__(64 * MERGE_WAVES) void attn_masked_decode_merge_kernel(DecodeArgs a) {
    constexpr int DV = VT_VALUE_DIM;
    __shared__ float ws_all[MERGE_WAVES][64];
    float* ws = ws_all[threadIdx.x >> 6];       // (every wave works the weights out for itself: no barrier)
    const int h = blockIdx.x, t = blockIdx.y, lane = threadIdx.x & 63;
    const int group = a.H / a.G;
    const int kvh = h / group, within = h % group;
    const int tile = kvh * a.HT + within / 16, r = within % 16;
    const float* base = a.part + ((((size_t)t * a.G * a.HT + tile) * a.P) * 16 + r) * DEC_ROW;
    const size_t step = (size_t)16 * DEC_ROW;
    const float LOG2E = 1.4426950408889634f;
    float mp = -INFINITY, lp = 0.f;
    if (lane < a.P) {
        mp = base[lane * step + DV];
        lp = base[lane * step + DV + 1];
    }
    float m_all = wave_max(mp);
    float extra = 0.f;
    if (a.sink && !a.sigmoid_weights) {
        // the sink is one more score with no value behind it
        const float sk = a.sink[h] * LOG2E;
        const float top = fmaxf(m_all, sk);
        extra = __builtin_amdgcn_exp2f(sk - top);
        m_all = top;
    }
    const float w = mp == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mp - m_all);
    float l = wave_sum(lp * w) + extra;
    if (a.sigmoid_weights) l = 1.f;             // (the parts' maxima are all 0 or none: every weight is 1)
    ws[lane] = w;
    wave_lds_order();
    const float f = ((a.gate && !a.gate_wide) ? gate_at(a.gate, a.gate_f32, a.ldg, t, h) : 1.f) / l;
    bf16_t* o = a.out + ((size_t)t * a.H + h) * DV;
    const int d = threadIdx.x;                  // a wave per 64 value elements
    if (d < DV) {
        float sum = 0.f;
#pragma unroll 8
        for (int p = 0; p < a.P; ++p) sum = fmaf(base[p * step + d], ws[p], sum);
        const float g = (a.gate && a.gate_wide) ? gate_at(a.gate, a.gate_f32, a.ldg, t, (size_t)h * DV + d) : 1.f;
        o[d] = f32_to_bf16(sum * f * g);
    }
}

extern "C" int vt_attn_masked_decode(const void* q, const void* k_pages, const void* v_pages, const int* positions,
                                     const int* tok_entry, const int* block_table, const void* gate, int gate_dtype,
                                     long long ldg, void* out, float* part, long long part_floats, int splits, int n,
                                     int H, int G, int D, int Dv, int page_size, int max_blocks, int num_pages, int window,
                                     int chunk, float scale, float cap, const float* sink, const float* slopes,
                                     const float* dist_r1, const float* dist_r2, const float* score_shift,
                                     int sigmoid_weights, int gate_wide, hipStream_t stream) {
    VT_REQUIRE((dist_r1 == nullptr) == (dist_r2 == nullptr), "vt_attn_masked_decode: the distance bias takes both of its numbers");
    VT_REQUIRE(!(sigmoid_weights && sink), "vt_attn_masked_decode: sigmoid weights have no denominator for a sink to join");
    VT_REQUIRE(!gate_wide || !gate || ldg >= (long long)H * Dv, "vt_attn_masked_decode: gate rows are too short");
    VT_REQUIRE(D == VT_KEY_DIM && Dv == VT_VALUE_DIM, "vt_attn_masked_decode: built for heads of %d/%d, called with %d/%d",
               VT_KEY_DIM, VT_VALUE_DIM, D, Dv);
    VT_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0, "vt_attn_masked_decode: bad heads %d/%d", H, G);
    VT_REQUIRE(page_size > 0 && page_size % 16 == 0 && max_blocks > 0 && num_pages > 0,
               "vt_attn_masked_decode: pages of %d keys (a multiple of 16)", page_size);
    VT_REQUIRE(window >= 0 && chunk >= 0 && cap >= 0.f, "vt_attn_masked_decode: bad mask or cap");
    VT_REQUIRE(splits >= 1 && splits <= 64, "vt_attn_masked_decode: %d splits (1 to 64)", splits);
    VT_REQUIRE(!gate || gate_dtype == VT_F32 || gate_dtype == VT_BF16, "vt_attn_masked_decode: gate dtype %d", gate_dtype);
    if (n == 0) return 0;
    const int HT = (H / G + 15) / 16;
    VT_REQUIRE(n <= 65535 && G * HT <= 65535 && H <= 65535, "vt_attn_masked_decode: too many tokens or heads");
    const long long need = (long long)n * G * HT * 4 * splits * 16 * DEC_ROW;
    VT_REQUIRE(part && part_floats >= need && (((uintptr_t)part) & 15) == 0,
               "vt_attn_masked_decode: %lld floats of scratch memory, %lld needed (16-byte aligned)", part_floats, need);
    DecodeArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages; a.positions = positions;
    a.tok_entry = tok_entry; a.block_table = block_table; a.sink = sink; a.slopes = slopes; a.gate = gate; a.part = part;
    a.out = (bf16_t*)out; a.ldg = ldg; a.n = n; a.H = H; a.G = G; a.HT = HT; a.P = 4 * splits; a.page_size = page_size;
    a.max_blocks = max_blocks; a.num_pages = num_pages; a.window = window; a.chunk = chunk; a.gate_f32 = gate_dtype == VT_F32;
    a.scale = scale; a.cap = cap; a.dist_r1 = dist_r1; a.dist_r2 = dist_r2; a.score_shift = score_shift;
    a.sigmoid_weights = sigmoid_weights; a.gate_wide = gate_wide;
    attn_masked_decode_kernel<<<dim3(splits, G * HT, n), 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_masked_decode");
    attn_masked_decode_merge_kernel<<<dim3(H, n), 64 * MERGE_WAVES, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_masked_decode(merge)");
    return 0;
}

extern "C" long long vt_attn_masked_decode_scratch(int n, int H, int G, int splits) {
    return (long long)n * G * ((H / G + 15) / 16) * 4 * splits * 16 * DEC_ROW;
}

extern "C" int vt_attn_masked_mfma_dims(int* key_dim, int* value_dim) {
    *key_dim = VT_KEY_DIM;
    *value_dim = VT_VALUE_DIM;
    return 0;
}

extern "C" int vt_attn_masked_mfma(const void* q, const void* k_pages, const void* v_pages, const int* positions,
                                   const int* tok_entry, const int* block_table, const int* tiles, int n_tiles,
                                   const void* gate, int gate_dtype, long long ldg, void* out, int H, int G, int D, int Dv,
                                   int page_size, int max_blocks, int num_pages, int window, int chunk, float scale,
                                   float cap, const float* sink, const float* slopes, const float* dist_r1,
                                   const float* dist_r2, const float* score_shift, int sigmoid_weights, int gate_wide,
                                   hipStream_t stream) {
    VT_REQUIRE((dist_r1 == nullptr) == (dist_r2 == nullptr), "vt_attn_masked_mfma: the distance bias takes both of its numbers");
    VT_REQUIRE(!(sigmoid_weights && sink), "vt_attn_masked_mfma: sigmoid weights have no denominator for a sink to join");
    VT_REQUIRE(!gate_wide || !gate || ldg >= (long long)H * Dv, "vt_attn_masked_mfma: gate rows are too short");
    VT_REQUIRE(D == VT_KEY_DIM && Dv == VT_VALUE_DIM, "vt_attn_masked_mfma: built for heads of %d/%d, called with %d/%d",
               VT_KEY_DIM, VT_VALUE_DIM, D, Dv);
    VT_REQUIRE(n_tiles >= 0 && H > 0 && G > 0 && H % G == 0, "vt_attn_masked_mfma: bad heads %d/%d", H, G);
    VT_REQUIRE(page_size > 0 && page_size % 16 == 0 && max_blocks > 0 && num_pages > 0,
               "vt_attn_masked_mfma: pages of %d keys (a multiple of 16)", page_size);
    VT_REQUIRE(window >= 0 && chunk >= 0 && cap >= 0.f, "vt_attn_masked_mfma: bad mask or cap");
    VT_REQUIRE(!gate || gate_dtype == VT_F32 || gate_dtype == VT_BF16, "vt_attn_masked_mfma: gate dtype %d", gate_dtype);
    if (n_tiles == 0) return 0;
    MfmaArgs a;
    a.q = (const bf16_t*)q; a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages; a.positions = positions;
    a.tok_entry = tok_entry; a.block_table = block_table; a.tiles = tiles; a.gate = gate; a.out = (bf16_t*)out; a.ldg = ldg;
    a.n_tiles = n_tiles; a.H = H; a.G = G; a.page_size = page_size; a.max_blocks = max_blocks; a.num_pages = num_pages;
    a.window = window; a.chunk = chunk; a.gate_f32 = gate_dtype == VT_F32; a.scale = scale; a.cap = cap;
    a.sink = sink; a.slopes = slopes; a.dist_r1 = dist_r1; a.dist_r2 = dist_r2; a.score_shift = score_shift;
    a.sigmoid_weights = sigmoid_weights; a.gate_wide = gate_wide;
    const long long items = (long long)n_tiles * H;
    if ((H / G) % 4 == 0)       // four heads of one key/value group to a block: they share what they read
        attn_masked_mfma_shared_kernel<<<(unsigned)(items / 4), 256, 0, stream>>>(a);
    else
        attn_masked_mfma_kernel<<<(unsigned)((items + 3) / 4), 256, 0, stream>>>(a);
    VT_CHECK_LAUNCH("vt_attn_masked_mfma");
    return 0;
}
