// Attention over paged keys and values for mixers whose heads the other attention kernels do not take: keys and
// values of different sizes, part of the head rotated, queries and keys scaled to unit root mean square, scores
// capped by a tanh, keys masked by a window or by chunks of positions, one gate per head.  Two kernels for prompts
// and decoding alike, in float32 or with 16-bit queries and pages; scores, softmax and sums are float32 in both.
//
//   vt_qk_prepare:  per token, rotate the leading `rot` elements of every query and key head (element i with element
//                   i + rot/2, angles from a table by position), divide by the head's root mean square if asked,
//                   write the queries out and keys and values into their pages:
//                   K [page][kv head][slot][D], V [page][kv head][Dv][slot].
//   vt_attn_masked: one block per (token, query head); keys are visited in chunks of 256 at absolute key indices
//                   with a running maximum and sum, so a token's result depends only on its position and the keys,
//                   not on how its request was cut into steps or what else is in the batch.
//                   score = cap * tanh(scale * q.k / cap) (cap 0: none); key j is seen from position i if j <= i,
//                   i - j < window (window 0: no bound) and j >= floor(i / chunk) * chunk (chunk 0: no bound);
//                   out = softmax(score) V * sigmoid(gate[token][head]) (no gate pointer: no gate).
//                   With `slopes`, slopes[head] * (i - j) is taken off the score of key j (behind the cap); with
//                   `sink`, exp(sink[head]) joins the softmax's denominator and nothing else: a key that holds no
//                   value.
//   vt_qk_prepare also scales the queries of position p by 1 + coef * ln(floor((p + 1) / every) + 1) (every 0: not),
//                   and mixes values across layers: vmix 1 leaves the token's values in `v_first` (float32), vmix 2
//                   writes (1 - lambda) v + lambda v_first into the pages instead of v.  With `q_gain` / `k_gain`
//                   ([D], shared by the heads) the unit-RMS queries / keys are multiplied by a gain per element.
//   vt_attn_masked, further forms of the score and of the weights, each switched on by its pointer or flag:
//                   `dist_r1`, `dist_r2` ([H] each): r1[head] * ln(1 + r2[head] * (i - j)) is taken off the score;
//                   `score_shift` ([H]): a number per head is added to every score;
//                   sigmoid_weights: the weight of a seen key is sigmoid(score) and nothing is normalized (no
//                   maximum, no sum, no sink); gate_wide: the gate is one logit per output element,
//                   gate[token][head * Dv + d], instead of one per head.
#include "vt_common.h"
#include <math.h>

VT_DEFINE_LAST_ERROR()

// ---------------------------------------------------------------------------
struct PrepArgs {
    const void* x;          // [n][ldx]: q heads, k heads, v heads, one after the other, from column 0
    const float* cos_t;     // [max_pos][rot/2]
    const float* sin_t;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    void* q_out;            // [n][H][D]
    void* k_pages;
    void* v_pages;
    long long ldx;
    int H, G, D, Dv, rot, max_pos, page_size, max_blocks, num_pages, write_kv, unit_rms;
    float eps;
    float q_temp_coef;      // queries times 1 + coef * ln(floor((pos + 1) / every) + 1); every 0: no factor
    int q_temp_every;
    int vmix;               // 0: none; 1: the values go to v_first as well; 2: the pages get (1 - lambda) v + lambda v_first
    float* v_first;         // [n][G * Dv] float32
    const float* v_lambda;  // one float on the device
    const float* q_gain;    // [D] or null: a gain per element on the unit-RMS queries
    const float* k_gain;    // [D] or null: likewise for the keys
};

template <typename TI, typename TC>
__global__ __launch_bounds__(256) void qk_prepare_kernel(PrepArgs a) {
    const int t = blockIdx.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
    const TI* x = (const TI*)a.x + (size_t)t * a.ldx;
    const int pos = a.positions[t];
    const int half = a.rot / 2;
    const float* c = a.cos_t + (size_t)pos * half;
    const float* s = a.sin_t + (size_t)pos * half;
    size_t page_row = 0;
    int page_no = 0, page_slot = 0;
    bool page_ok = false;
    if (a.write_kv) {
        const int blk = pos / a.page_size;
        const int pg = blk < a.max_blocks ? a.block_table[(size_t)a.tok_entry[t] * a.max_blocks + blk] : -1;
        page_ok = pg >= 0 && pg < a.num_pages;
        page_no = page_ok ? pg : 0;
        page_slot = pos - blk * a.page_size;
        page_row = (size_t)page_no * a.G * a.page_size + page_slot;
    }
    const int units = a.H + (a.write_kv ? 2 * a.G : 0);
    for (int u = blockIdx.y * nw + wave; u < units; u += nw * gridDim.y) {
        if (u < a.H + a.G) {
            // a query or key head: rotate, then scale to unit root mean square
            const bool is_q = u < a.H;
            const TI* src = x + (size_t)u * a.D;
            float vals[4];      // D <= 256: up to four elements per lane
            float ss = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = lane + 64 * i;
                float v = 0.f;
                if (d < a.D) {
                    v = load_f32<TI>(src, d);
                    if (d < a.rot && pos < a.max_pos) {
                        const bool low = d < half;
                        const int p = low ? d : d - half;
                        const float y = load_f32<TI>(src, low ? d + half : d - half);
                        v = rotate_pair(c[p], s[p], v, y, low);
                    }
                }
                vals[i] = v;
                ss += v * v;
            }
            float r = 1.f;
            if (a.unit_rms) {
                ss = wave_sum(ss);
                r = 1.0f / sqrtf(ss / (float)a.D + a.eps);
            }
            if (is_q && a.q_temp_every > 0) r *= 1.0f + a.q_temp_coef * logf((float)((pos + 1) / a.q_temp_every) + 1.0f);
            const float* gain = is_q ? a.q_gain : a.k_gain;
            if (gain) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = lane + 64 * i;
                    if (d < a.D) vals[i] = vals[i] * r * gain[d];
                }
                r = 1.f;
            }
            if (is_q) {
                TC* dst = (TC*)a.q_out + ((size_t)t * a.H + u) * a.D;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = lane + 64 * i;
                    if (d < a.D) store_f32<TC>(dst, d, vals[i] * r);
                }
            } else if (page_ok) {
                const int g = u - a.H;
                TC* dst = (TC*)a.k_pages + (page_row + (size_t)g * a.page_size) * a.D;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int d = lane + 64 * i;
                    if (d < a.D) store_f32<TC>(dst, d, vals[i] * r);
                }
            }
        } else if (page_ok) {
            // values transposed inside the page, [kv head][Dv][slot]: the matrix-core kernel reads keys four at a time
            const int g = u - a.H - a.G;
            const TI* src = x + (size_t)(a.H + a.G) * a.D + (size_t)g * a.Dv;
            TC* dst = (TC*)a.v_pages + ((size_t)page_no * a.G + g) * a.Dv * a.page_size + page_slot;
            float* vf = a.v_first + ((size_t)t * a.G + g) * a.Dv;
            const float lam = a.vmix == 2 ? a.v_lambda[0] : 0.f;
            for (int d = lane; d < a.Dv; d += 64) {
                float v = load_f32<TI>(src, d);
                if (a.vmix == 1) vf[d] = v;
                else if (a.vmix == 2) v = (1.0f - lam) * v + lam * vf[d];
                store_f32<TC>(dst, (size_t)d * a.page_size, v);
            }
        }
    }
}

extern "C" int vt_qk_prepare(const void* x, int x_dtype, long long ldx, const float* cos_t, const float* sin_t, int rot,
                             int max_pos, const int* positions, const int* tok_entry, const int* block_table,
                             int max_blocks, void* q_out, void* k_pages, void* v_pages, int cache_dtype, int page_size,
                             int num_pages, int n, int H, int G, int D, int Dv, int write_kv, int unit_rms, float eps,
                             float q_temp_coef, int q_temp_every, int vmix, float* v_first, const float* v_lambda,
                             const float* q_gain, const float* k_gain, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0, "vt_qk_prepare: bad heads %d/%d", H, G);
    VT_REQUIRE(D > 0 && D <= 256 && Dv > 0, "vt_qk_prepare: head sizes %d/%d (keys up to 256)", D, Dv);
    VT_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D, "vt_qk_prepare: %d rotated elements of %d", rot, D);
    VT_REQUIRE(rot == 0 || (cos_t && sin_t && max_pos > 0), "vt_qk_prepare: no table of angles");
    VT_REQUIRE(ldx >= (long long)(H + (write_kv ? G : 0)) * D + (write_kv ? (long long)G * Dv : 0),
               "vt_qk_prepare: rows of %lld elements are too short", ldx);
    VT_REQUIRE(!write_kv || (page_size > 0 && max_blocks > 0 && num_pages > 0 && block_table && k_pages && v_pages),
               "vt_qk_prepare: bad cache sizes");
    VT_REQUIRE(q_temp_every >= 0, "vt_qk_prepare: a query factor every %d positions", q_temp_every);
    VT_REQUIRE(vmix == 0 || ((vmix == 1 || vmix == 2) && write_kv && v_first && (vmix == 1 || v_lambda)),
               "vt_qk_prepare: value mixing %d without its buffers", vmix);
    if (n == 0) return 0;
    PrepArgs a;
    a.x = x; a.cos_t = cos_t; a.sin_t = sin_t; a.positions = positions; a.tok_entry = tok_entry; a.block_table = block_table;
    a.q_out = q_out; a.k_pages = k_pages; a.v_pages = v_pages; a.ldx = ldx; a.H = H; a.G = G; a.D = D; a.Dv = Dv; a.rot = rot;
    a.max_pos = max_pos; a.page_size = page_size; a.max_blocks = max_blocks; a.num_pages = num_pages; a.write_kv = write_kv;
    a.unit_rms = unit_rms; a.eps = eps; a.q_temp_coef = q_temp_coef; a.q_temp_every = q_temp_every; a.vmix = vmix;
    a.v_first = v_first; a.v_lambda = v_lambda; a.q_gain = q_gain; a.k_gain = k_gain;
    // few tokens: a wave per head, over several blocks per token; many tokens: a block per token goes through its heads
    const int units = H + (write_kv ? 2 * G : 0);
    const dim3 grid(n, n >= 1024 ? 1 : (units + 3) / 4);
    if (x_dtype == VT_F32 && cache_dtype == VT_F32) qk_prepare_kernel<float, float><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_F32 && cache_dtype == VT_BF16) qk_prepare_kernel<float, bf16_t><<<grid, 256, 0, stream>>>(a);
    else if (x_dtype == VT_BF16 && cache_dtype == VT_BF16) qk_prepare_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>(a);
    else return vt_fail("vt_qk_prepare: dtypes %d -> %d are not handled", x_dtype, cache_dtype);
    VT_CHECK_LAUNCH("vt_qk_prepare");
    return 0;
}

// ---------------------------------------------------------------------------
struct MaskedArgs {
    const void* q;
    const void* k_pages;
    const void* v_pages;
    const int* positions;
    const int* tok_entry;
    const int* block_table;
    const void* gate;       // gate[t * ldg + h], or null
    const float* sink;      // [H], or null: exp(sink[h]) joins the denominator
    const float* slopes;    // [H], or null: slopes[h] * (position - key index) is taken off every score
    const float* dist_r1;   // [H] each, or null: r1[h] * ln(1 + r2[h] * (position - key index)) is taken off every score
    const float* dist_r2;
    const float* score_shift;   // [H], or null: added to every score
    void* out;              // [n][H][Dv]
    long long ldg;
    int sigmoid_weights;    // 1: weight = sigmoid(score), not normalized
    int gate_wide;          // 1: gate[t * ldg + h * Dv + d]
    int H, G, D, Dv, page_size, max_blocks, num_pages, window, chunk;
    float scale, cap;
};

#define KEYS 256

template <typename TC, typename TG>
__global__ __launch_bounds__(KEYS) void attn_masked_kernel(MaskedArgs a) {
    extern __shared__ float smem[];
    float* qs = smem;             // D
    float* sp = qs + a.D;         // KEYS
    float* spart = sp + KEYS;     // KEYS
    __shared__ float red[16];

    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int D = a.D, Dv = a.Dv, ps = a.page_size;
    const int kvh = h / (a.H / a.G);
    const int pos = a.positions[t];
    const int* bt = a.block_table + (size_t)a.tok_entry[t] * a.max_blocks;
    int lo = a.chunk > 0 ? (pos / a.chunk) * a.chunk : 0;
    if (a.window > 0) lo = max(lo, pos - a.window + 1);
    const TC* kp = (const TC*)a.k_pages;
    const TC* vp = (const TC*)a.v_pages;
    const float slope = a.slopes ? a.slopes[h] : 0.f;
    const float r1 = a.dist_r1 ? a.dist_r1[h] : 0.f, r2 = a.dist_r1 ? a.dist_r2[h] : 0.f;
    const float shift = a.score_shift ? a.score_shift[h] : 0.f;
    const bool sig = a.sigmoid_weights != 0;

    for (int d = tid; d < D; d += KEYS) qs[d] = load_f32<TC>((const TC*)a.q, ((size_t)t * a.H + h) * D + d);
    __syncthreads();

    const bool wide = Dv > KEYS;  // value heads wider than the block: a thread takes columns tid, tid + KEYS, ... (up to 4)
    const int Gv = wide ? 1 : KEYS / Dv;     // key groups for the weighted sum
    const int d_own = wide ? tid : tid % Dv, g_own = wide ? 0 : tid / Dv;
    const bool pv_active = g_own < Gv;

    float m = -INFINITY, l = 0.f, acc = 0.f;
    float acc_w[3] = {0.f, 0.f, 0.f};        // columns tid + KEYS, tid + 2 KEYS, tid + 3 KEYS of a wide head
    for (int c0 = (lo / KEYS) * KEYS; c0 <= pos; c0 += KEYS) {
        const int j = c0 + tid;
        const bool valid = j >= lo && j <= pos;
        float s = -INFINITY;
        if (valid) {
            const int blk = j / ps;
            const int pg = bt[blk];
            if (pg >= 0 && pg < a.num_pages) {
                const TC* kr = kp + (((size_t)pg * a.G + kvh) * ps + (j - blk * ps)) * D;
                float dot = 0.f;
                for (int d = 0; d < D; ++d) dot = fmaf(qs[d], load_f32<TC>(kr, d), dot);
                s = dot * a.scale;
                if (a.cap > 0.f) s = a.cap * tanhf(s / a.cap);
                if (a.slopes) s -= slope * (float)(pos - j);
                if (a.dist_r1) s -= r1 * log1pf(r2 * (float)(pos - j));
                s += shift;
            } else {
                s = __int_as_float(0x7fc00000);  // a missing page must show, not pass as a masked key
            }
        }
        float m_new = 0.f, alpha = 1.f;
        if (sig) {
            // every key's weight stands alone: nothing to rescale
            sp[tid] = valid ? 1.0f / (1.0f + expf(-s)) : 0.f;
            __syncthreads();
        } else {
            const float cmax = block_max(s, red);
            m_new = fmaxf(m, cmax);
            const float p = valid ? expf(s - m_new) : 0.f;
            sp[tid] = p;
            const float csum = block_sum(p, red);  // its barriers also publish sp
            alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
            l = l * alpha + csum;
        }

        float part = 0.f;
        if (pv_active) {
            for (int jj = g_own; jj < KEYS; jj += Gv) {
                const int jk = c0 + jj;
                if (jk < lo || jk > pos) continue;
                const int blk = jk / ps;
                const int pg = bt[blk];
                if (pg < 0 || pg >= a.num_pages) continue;
                part = fmaf(sp[jj], load_f32<TC>(vp, (((size_t)pg * a.G + kvh) * Dv + d_own) * ps + (jk - blk * ps)), part);
            }
        }
        if (wide) {
#pragma unroll
            for (int c = 1; c < 4; ++c) {
                const int d = tid + c * KEYS;
                if (d >= Dv) break;
                float pw = 0.f;
                for (int jj = 0; jj < KEYS; ++jj) {
                    const int jk = c0 + jj;
                    if (jk < lo || jk > pos) continue;
                    const int blk = jk / ps;
                    const int pg = bt[blk];
                    if (pg < 0 || pg >= a.num_pages) continue;
                    pw = fmaf(sp[jj], load_f32<TC>(vp, (((size_t)pg * a.G + kvh) * Dv + d) * ps + (jk - blk * ps)), pw);
                }
                acc_w[c - 1] = acc_w[c - 1] * alpha + pw;
            }
        }
        spart[tid] = part;
        __syncthreads();
        if (tid < Dv) {
            float sum = 0.f;
            for (int g = 0; g < Gv; ++g) sum += spart[g * Dv + tid];
            acc = acc * alpha + sum;
        }
        __syncthreads();
        m = m_new;
    }
    if (sig) l = 1.f;
    if (a.sink && !sig) {
        // the sink is one more score with no value behind it
        const float sk = a.sink[h];
        const float m_all = fmaxf(m, sk);
        const float keep = expf(m - m_all);
        l = l * keep + expf(sk - m_all);
        acc *= keep;
#pragma unroll
        for (int c = 0; c < 3; ++c) acc_w[c] *= keep;
    }
    // the gate's logit of output element d: one per head, or one per element
    auto gate_of = [&](int d) -> float {
        if (!a.gate) return 1.f;
        const float z = load_f32<TG>((const TG*)a.gate, (size_t)t * a.ldg + (a.gate_wide ? (size_t)h * Dv + d : (size_t)h));
        return 1.0f / (1.0f + expf(-z));
    };
    if (tid < Dv) store_f32<TC>((TC*)a.out, ((size_t)t * a.H + h) * Dv + tid, (acc / l) * gate_of(tid));
    if (wide) {
#pragma unroll
        for (int c = 1; c < 4; ++c)
            if (tid + c * KEYS < Dv)
                store_f32<TC>((TC*)a.out, ((size_t)t * a.H + h) * Dv + tid + c * KEYS, acc_w[c - 1] * (gate_of(tid + c * KEYS) / l));
    }
}

extern "C" int vt_attn_masked(const void* q, const void* k_pages, const void* v_pages, int dtype, const int* positions,
                              const int* tok_entry, const int* block_table, const void* gate, int gate_dtype,
                              long long ldg, void* out, int n, int H, int G, int D, int Dv, int page_size,
                              int max_blocks, int num_pages, int window, int chunk, float scale, float cap,
                              const float* sink, const float* slopes, const float* dist_r1, const float* dist_r2,
                              const float* score_shift, int sigmoid_weights, int gate_wide, hipStream_t stream) {
    VT_REQUIRE(n >= 0 && H > 0 && G > 0 && H % G == 0, "vt_attn_masked: bad heads %d/%d", H, G);
    VT_REQUIRE((dist_r1 == nullptr) == (dist_r2 == nullptr), "vt_attn_masked: the distance bias takes both of its numbers");
    VT_REQUIRE(!(sigmoid_weights && sink), "vt_attn_masked: sigmoid weights have no denominator for a sink to join");
    VT_REQUIRE(!gate_wide || ldg >= (long long)H * Dv, "vt_attn_masked: gate rows are too short");
    VT_REQUIRE(D > 0 && D <= 8192 && Dv > 0 && Dv <= 4 * KEYS, "vt_attn_masked: head sizes %d/%d (keys up to 8192, values up to %d)", D, Dv, 4 * KEYS);
    VT_REQUIRE(page_size > 0 && max_blocks > 0 && num_pages > 0, "vt_attn_masked: bad cache sizes");
    VT_REQUIRE(H <= 65535, "vt_attn_masked: too many heads (%d)", H);
    VT_REQUIRE(window >= 0 && chunk >= 0 && cap >= 0.f, "vt_attn_masked: bad mask or cap");
    if (n == 0) return 0;
    MaskedArgs a;
    a.q = q; a.k_pages = k_pages; a.v_pages = v_pages; a.positions = positions; a.tok_entry = tok_entry;
    a.block_table = block_table; a.gate = gate; a.out = out; a.ldg = ldg; a.H = H; a.G = G; a.D = D; a.Dv = Dv;
    a.page_size = page_size; a.max_blocks = max_blocks; a.num_pages = num_pages; a.window = window; a.chunk = chunk;
    a.scale = scale; a.cap = cap; a.sink = sink; a.slopes = slopes; a.dist_r1 = dist_r1; a.dist_r2 = dist_r2;
    a.score_shift = score_shift; a.sigmoid_weights = sigmoid_weights; a.gate_wide = gate_wide;
    const size_t shmem = (size_t)(D + 2 * KEYS) * sizeof(float);
    const dim3 grid(n, H);
    if (dtype == VT_F32) {
        VT_REQUIRE(!gate || gate_dtype == VT_F32, "vt_attn_masked: float32 takes float32 gates");
        attn_masked_kernel<float, float><<<grid, KEYS, shmem, stream>>>(a);
    } else if (dtype == VT_BF16) {
        if (gate && gate_dtype == VT_BF16) attn_masked_kernel<bf16_t, bf16_t><<<grid, KEYS, shmem, stream>>>(a);
        else attn_masked_kernel<bf16_t, float><<<grid, KEYS, shmem, stream>>>(a);
    } else {
        return vt_fail("vt_attn_masked: unknown dtype %d", dtype);
    }
    VT_CHECK_LAUNCH("vt_attn_masked");
    return 0;
}
