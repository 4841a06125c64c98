// Attention whose heads exchange their scores before the softmax, over the paged cache:
//
//   s_g(i, j) = cap * tanh(scale * q_g(i) . k_g(j) / cap)  [cap > 0]  + bias[min(i - j, rows - 1), g]
//   s'_h(i, j) = sum_g mix[h, g] * s_g(i, j)                         [mix given]
//   visible: j <= i and (i - j < window or j < keep_first)           [window > 0; else all j <= i]
//   p_h(i, j) = exp(s'_h) / (sink + sum over visible j of exp(s'_h))  (sink = 1: a key of score 0 without a value)
//   out_h(i) = sum_j p_h(i, j) v(j)
//
// Query head g reads kv head g / (H / G).  Scores, bias, mixing and softmax are float32.  Keys lie
// in pages [kv head, slot, element], values transposed [kv head, element, slot].
//
// tff_qk_bias_norm_store: q and k rows from one projection [T, (H + G) * D] (float32) get their biases;
//   q is divided by its root mean square over the head and written out; k goes into the token's slot
//   twice: as projected into the value page, divided by its root mean square into the key page.
// tff_mixed_attention: one block per query token, all heads; keys in tiles of 64 whose borders are
//   multiples of 64 from the sequence's start, so a query's sums are formed in the same order in
//   every step that computes it.
#include "common.h"
#include "tffinfer_kernels.h"

template <typename TC>
__global__ __launch_bounds__(256) void qk_bias_norm_store_kernel(
    const float* __restrict__ qk, size_t row, const float* __restrict__ qb, const float* __restrict__ kb, float eps,
    TC* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const int32_t* __restrict__ slot_mapping, int page_size, int pairs, int H, int G, int D) {
    const int id = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (id >= pairs) return;
    const int t = id / (H + G), head = id % (H + G);
    const float* src = qk + (size_t)t * row + (size_t)head * D;
    const float* bias = head < H ? (qb ? qb + (size_t)head * D : nullptr) : (kb ? kb + (size_t)(head - H) * D : nullptr);
    float ss = 0.f;
    for (int e = lane; e < D; e += 64) {
        const float a = src[e] + (bias ? bias[e] : 0.f);
        ss = fmaf(a, a, ss);
    }
    ss = wave_sum(ss);
    const float rr = 1.0f / sqrtf(ss / (float)D + eps);
    if (head < H) {
        TC* dst = q_out + ((size_t)t * H + head) * D;
        for (int e = lane; e < D; e += 64) dst[e] = from_f32<TC>((src[e] + (bias ? bias[e] : 0.f)) * rr);
        return;
    }
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    const int g = head - H, page = slot / page_size, off = slot % page_size;
    TC* kd = k_cache + (((size_t)page * G + g) * page_size + off) * D;
    TC* vd = v_cache + ((size_t)page * G + g) * D * page_size + off;
    for (int e = lane; e < D; e += 64) {
        const float a = src[e] + (bias ? bias[e] : 0.f);
        kd[e] = from_f32<TC>(a * rr);
        vd[(size_t)e * page_size] = from_f32<TC>(a);
    }
}

TFF_API int tff_qk_bias_norm_store(const float* qk, size_t row, const float* qb, const float* kb, float eps, void* q_out,
                                   void* k_cache, void* v_cache, const int32_t* slot_mapping, int page_size, int T, int H,
                                   int G, int D, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(qk && q_out && k_cache && v_cache && slot_mapping, "qk_bias_norm_store: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && page_size > 0 && row >= (size_t)(H + G) * D,
                "qk_bias_norm_store: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int pairs = T * (H + G);
    if (dtype == TFF_F32)
        qk_bias_norm_store_kernel<float><<<(pairs + 3) / 4, 256, 0, s>>>(qk, row, qb, kb, eps, (float*)q_out, (float*)k_cache,
                                                                         (float*)v_cache, slot_mapping, page_size, pairs, H, G, D);
    else if (dtype == TFF_BF16)
        qk_bias_norm_store_kernel<bf16_t><<<(pairs + 3) / 4, 256, 0, s>>>(qk, row, qb, kb, eps, (bf16_t*)q_out,
                                                                          (bf16_t*)k_cache, (bf16_t*)v_cache, slot_mapping,
                                                                          page_size, pairs, H, G, D);
    else
        return tff_fail("qk_bias_norm_store: unknown dtype %d", dtype);
    return tff_check_launch("qk_bias_norm_store");
}

#define MA_TK 64        // keys a tile: one a lane where a wave takes a head's scores
#define MA_THREADS 256
#define MA_WAVES 4

// eight consecutive elements as floats
__device__ __forceinline__ void ma_load8(const float* p, float* f) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}
__device__ __forceinline__ void ma_load8(const bf16_t* p, float* f) {
    union { uint4 u; bf16_t h[8]; } pk;
    pk.u = *reinterpret_cast<const uint4*>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) f[i] = (float)pk.h[i];
}

template <typename TC, int ACC>
__global__ __launch_bounds__(MA_THREADS) void mixed_attention_kernel(
    const TC* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int bt_width, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ positions, const float* __restrict__ bias, int bias_rows,
    const float* __restrict__ mix, float scale, float cap, int window, int keep_first, int sink,
    TC* __restrict__ out, int H, int G, int D, int page_size) {
    extern __shared__ float lds[];
    float* q_s = lds;                       // [H][D]
    float* s_raw = q_s + H * D;             // [H][TK]
    float* p_s = s_raw + H * MA_TK;         // [H][TK]
    float* mix_s = p_s + H * MA_TK;         // [H][H] (if mix)
    float* m_s = mix_s + (mix ? H * H : 0); // [H]
    float* l_s = m_s + H;
    float* c_s = l_s + H;
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int pos = positions[t];
    const int32_t* table = block_tables + (size_t)token_req[t] * bt_width;
    const int rep = H / G, HD = H * D;
    const bool vec = (D % 8) == 0;
    for (int i = tid; i < HD; i += MA_THREADS) q_s[i] = to_f32(q[(size_t)t * HD + i]);
    if (mix)
        for (int i = tid; i < H * H; i += MA_THREADS) mix_s[i] = mix[i];
    for (int i = tid; i < H; i += MA_THREADS) {
        m_s[i] = sink ? 0.f : -INFINITY;
        l_s[i] = sink ? 1.f : 0.f;
    }
    float acc[ACC];
#pragma unroll
    for (int n = 0; n < ACC; ++n) acc[n] = 0.f;
    __syncthreads();
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    // two ranges of keys: the first tokens that are kept (those the window does not hold anyway), and the window
    for (int range = 0; range < 2; ++range) {
        const int r_lo = range == 0 ? 0 : lo;
        const int r_hi = range == 0 ? min(keep_first, lo) : pos + 1;     // (exclusive)
        for (int jt = (r_lo / MA_TK) * MA_TK; jt < r_hi; jt += MA_TK) {
            // scores of all heads for the tile's keys
            {
                const int j = jt + lane;
                const bool vis = j >= r_lo && j < r_hi;
                if (vis) {
                    const int page = table[j / page_size], off = j % page_size;
                    const int dist = min(pos - j, bias_rows - 1);
                    for (int g = wv; g < H; g += MA_WAVES) {
                        const TC* kr = k_cache + (((size_t)page * G + g / rep) * page_size + off) * D;
                        const float* qg = q_s + g * D;
                        float dot = 0.f;
                        if (vec) {
                            for (int d = 0; d < D; d += 8) {
                                float kf[8];
                                ma_load8(kr + d, kf);
#pragma unroll
                                for (int e = 0; e < 8; ++e) dot = fmaf(qg[d + e], kf[e], dot);
                            }
                        } else {
                            for (int d = 0; d < D; ++d) dot = fmaf(qg[d], to_f32(kr[d]), dot);
                        }
                        float sc = dot * scale;
                        if (cap > 0.f) sc = cap * tanhf(sc / cap);
                        if (bias) sc += bias[(size_t)dist * H + g];
                        s_raw[g * MA_TK + lane] = sc;
                    }
                } else {
                    for (int g = wv; g < H; g += MA_WAVES) s_raw[g * MA_TK + lane] = 0.f;
                }
            }
            __syncthreads();
            // the heads' scores mixed; the running maximum and sum of each head, a wave a head
            {
                const int j = jt + lane;
                const bool vis = j >= r_lo && j < r_hi;
                for (int h = wv; h < H; h += MA_WAVES) {
                    float sc;
                    if (mix) {
                        sc = 0.f;
                        for (int g = 0; g < H; ++g) sc = fmaf(mix_s[h * H + g], s_raw[g * MA_TK + lane], sc);
                    } else {
                        sc = s_raw[h * MA_TK + lane];
                    }
                    if (!vis) sc = -INFINITY;
                    const float m_old = m_s[h];
                    const float m_new = fmaxf(m_old, wave_max(sc));
                    float p = 0.f, corr = 1.f;
                    if (m_new > -INFINITY) {
                        p = vis ? expf(sc - m_new) : 0.f;
                        corr = expf(m_old - m_new);
                    }
                    const float l_new = l_s[h] * corr + wave_sum(p);
                    p_s[h * MA_TK + lane] = p;
                    if (lane == 0) {
                        m_s[h] = m_new;
                        l_s[h] = l_new;
                        c_s[h] = corr;
                    }
                }
            }
            __syncthreads();
            // weighted values: thread -> (head, element) pairs
            {
                const int j_lo = max(jt, r_lo) & ~7, j_hi = min(jt + MA_TK, r_hi);
#pragma unroll
                for (int n = 0; n < ACC; ++n) {
                    const int idx = tid + n * MA_THREADS;
                    if (idx < HD) {
                        const int h = idx / D, e = idx % D;
                        float a = acc[n] * c_s[h];
                        const float* ph = p_s + h * MA_TK - jt;
                        for (int j = j_lo; j < j_hi; j += 8) {     // (pages hold a multiple of 8 tokens)
                            const int page = table[j / page_size], off = j % page_size;
                            const TC* vr = v_cache + (((size_t)page * G + h / rep) * D + e) * page_size + off;
                            float vf[8];
                            ma_load8(vr, vf);
#pragma unroll
                            for (int i = 0; i < 8; ++i) a = fmaf(ph[j + i], vf[i], a);
                        }
                        acc[n] = a;
                    }
                }
            }
            // (the next tile's scores go to s_raw, which nobody reads any more; its barrier stands
            // between these reads of p_s and the next writes)
        }
    }
    __syncthreads();
#pragma unroll
    for (int n = 0; n < ACC; ++n) {
        const int idx = tid + n * MA_THREADS;
        if (idx < HD) {
            const float l = l_s[idx / D];
            out[(size_t)t * HD + idx] = from_f32<TC>(l > 0.f ? acc[n] / l : 0.f);
        }
    }
}

static size_t ma_lds_bytes(int H, int D, bool mix) {
    return sizeof(float) * ((size_t)H * D + 2 * (size_t)H * MA_TK + (mix ? (size_t)H * H : 0) + 3 * (size_t)H);
}

TFF_API int tff_mixed_attention_supported(int H, int D, int has_mix) {
    return H > 0 && D > 0 && (size_t)H * D <= 16 * MA_THREADS && ma_lds_bytes(H, D, has_mix != 0) <= 64 * 1024;
}

template <typename TC>
static int ma_launch(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables, int bt_width,
                     const int32_t* token_req, const int32_t* positions, const float* bias, int bias_rows, const float* mix,
                     float scale, float cap, int window, int keep_first, int sink, void* out, int T, int H, int G, int D,
                     int page_size, hipStream_t s) {
    const size_t lds = ma_lds_bytes(H, D, mix != nullptr);
    const int per = (H * D + MA_THREADS - 1) / MA_THREADS;
#define MA_LAUNCH(ACC)                                                                                                   \
    mixed_attention_kernel<TC, ACC><<<T, MA_THREADS, lds, s>>>((const TC*)q, (const TC*)k_cache, (const TC*)v_cache,      \
                                                                block_tables, bt_width, token_req, positions, bias,      \
                                                                bias_rows, mix, scale, cap, window, keep_first, sink,    \
                                                                (TC*)out, H, G, D, page_size)
    if (per <= 1) MA_LAUNCH(1);
    else if (per <= 2) MA_LAUNCH(2);
    else if (per <= 4) MA_LAUNCH(4);
    else if (per <= 8) MA_LAUNCH(8);
    else MA_LAUNCH(16);
#undef MA_LAUNCH
    return tff_check_launch("mixed_attention");
}

TFF_API int tff_mixed_attention(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                int bt_width, const int32_t* token_req, const int32_t* positions, const float* bias,
                                int bias_rows, const float* mix, float scale, float cap, int window, int keep_first,
                                int sink, void* out, int T, int H, int G, int D, int page_size, int dtype,
                                tff_stream_t stream) {
    TFF_REQUIRE(q && k_cache && v_cache && block_tables && token_req && positions && out, "mixed_attention: null pointer");
    TFF_REQUIRE(T >= 0 && G > 0 && H % G == 0 && bt_width > 0 && page_size > 0 && page_size % 8 == 0,
                "mixed_attention: %d heads on %d kv heads, pages of %d", H, G, page_size);
    TFF_REQUIRE(tff_mixed_attention_supported(H, D, mix != nullptr), "mixed_attention: %d heads of %d do not fit a block", H, D);
    TFF_REQUIRE(!bias || bias_rows > 0, "mixed_attention: a bias table without rows");
    TFF_REQUIRE(window >= 0 && keep_first >= 0, "mixed_attention: negative window");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        return ma_launch<float>(q, k_cache, v_cache, block_tables, bt_width, token_req, positions, bias, bias_rows, mix,
                                scale, cap, window, keep_first, sink, out, T, H, G, D, page_size, s);
    if (dtype == TFF_BF16)
        return ma_launch<bf16_t>(q, k_cache, v_cache, block_tables, bt_width, token_req, positions, bias, bias_rows, mix,
                                 scale, cap, window, keep_first, sink, out, T, H, G, D, page_size, s);
    return tff_fail("mixed_attention: unknown dtype %d", dtype);
}
