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
// tff_mixed_attention: one block per query token (and split of its keys), all heads; keys in tiles of 64
//   whose borders are multiples of 64 from the sequence's start, so a query's sums are formed in the same
//   order in every step that computes it with the same number of splits; a step of few tokens splits each
//   token's tiles over several blocks and a second kernel puts them together.
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
#define MA_THREADS 512   // eight waves: two a SIMD, so that LDS and lane-swap latencies of one hide behind the other
#define MA_WAVES 8

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

// A token's visible keys lie in two ranges: the first tokens that are kept (those that the window does not
// hold anyway), [0, a_hi), and the window, [lo, pos].  Their tiles are numbered through: first those of
// the first range, then those of the second, each starting at a multiple of MA_TK.
struct MaTiles {
    int a_hi, lo, hi, n_a, jt_b, n;
    __device__ MaTiles(int pos, int window, int keep_first) {
        lo = window > 0 ? max(0, pos - window + 1) : 0;
        a_hi = min(keep_first, lo);
        hi = pos + 1;
        n_a = (a_hi + MA_TK - 1) / MA_TK;
        jt_b = (lo / MA_TK) * MA_TK;
        n = n_a + (pos - jt_b) / MA_TK + 1;
    }
};

// One block per (token, split of the token's tiles).  With one split the block writes the token's result;
// with more it leaves, per head, its running maximum, its sum and the unnormalised weighted values for
// mixed_attention_merge_kernel (the sink's term is then the merge's to add).
// Eight consecutive elements as they come from memory; several are asked for before the first is used, so that
// a thread waits for memory once per group and not once per load.
template <typename TC> struct MaRaw;
template <> struct MaRaw<bf16_t> {
    uint4 u;
    __device__ __forceinline__ void load(const bf16_t* p) { u = *reinterpret_cast<const uint4*>(p); }
    __device__ __forceinline__ void zero() { u = make_uint4(0, 0, 0, 0); }
    __device__ __forceinline__ void get(float* f) const {
        union { uint4 u; bf16_t h[8]; } pk;
        pk.u = u;
#pragma unroll
        for (int i = 0; i < 8; ++i) f[i] = (float)pk.h[i];
    }
};
template <> struct MaRaw<float> {
    float4 a, b;
    __device__ __forceinline__ void load(const float* p) {
        a = *reinterpret_cast<const float4*>(p);
        b = *reinterpret_cast<const float4*>(p + 4);
    }
    __device__ __forceinline__ void zero() { a = make_float4(0, 0, 0, 0); b = a; }
    __device__ __forceinline__ void get(float* f) const {
        f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
    }
};

#define MA_AHEAD 4      // key rows a wave asks for before it multiplies the first
#define MA_RUNS 4       // runs of 8 values a thread asks for before it multiplies the first

template <typename TC, int ACC>
__global__ __launch_bounds__(MA_THREADS) void mixed_attention_kernel(
    const TC* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int bt_width, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ positions, const float* __restrict__ bias, int bias_rows,
    const float* __restrict__ mix, float scale, float cap, int window, int keep_first, int sink,
    TC* __restrict__ out, int H, int G, int D, int page_size, int tiles_per_split, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
    extern __shared__ float lds[];
    float* q_s = lds;                       // [H][D]
    float* s_raw = q_s + H * D;             // [H][TK]
    float* p_s = s_raw + H * MA_TK;         // [H][TK]
    float* mix_s = p_s + H * MA_TK;         // [H][H] (if mix)
    float* m_s = mix_s + (mix ? H * H : 0); // [H]
    float* l_s = m_s + H;
    float* c_s = l_s + H;
    // per run of 8 keys of a tile: its page and its place in the page; two sets, by the tile's parity (a wave may
    // be at the next tile's products while another still weighs this tile's values)
    int* chunk_s = reinterpret_cast<int*>(c_s + H);      // [2][2][TK / 8]
    const int t = blockIdx.x, split = blockIdx.y, nsplit = gridDim.y;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
    const int pos = positions[t];
    const int32_t* table = block_tables + (size_t)token_req[t] * bt_width;
    const int rep = H / G, HD = H * D;
    const bool own_sink = sink && nsplit == 1;
    for (int i = tid; i < HD; i += MA_THREADS) q_s[i] = to_f32(q[(size_t)t * HD + i]);
    if (mix)
        for (int i = tid; i < H * H; i += MA_THREADS) mix_s[i] = mix[i];
    for (int i = tid; i < H; i += MA_THREADS) {
        m_s[i] = own_sink ? 0.f : -INFINITY;
        l_s[i] = own_sink ? 1.f : 0.f;
    }
    float acc[ACC];
#pragma unroll
    for (int n = 0; n < ACC; ++n) acc[n] = 0.f;
    __syncthreads();
    const MaTiles tiles(pos, window, keep_first);
    const int i_lo = nsplit == 1 ? 0 : split * tiles_per_split;
    const int i_hi = split == nsplit - 1 ? tiles.n : min(tiles.n, i_lo + tiles_per_split);      // (the last split takes what is left)
    // lanes of a key: a key's row of D elements is read by D / 8 neighbouring lanes, 16 bytes each (where D / 8
    // is a power of two up to 64), so that a wave's load covers whole rows; else a lane reads a key's whole row
    const int lpk = D / 8;
    const bool rows_by_lanes = D % 8 == 0 && lpk <= 64 && (lpk & (lpk - 1)) == 0;
    const int lpk_shift = 31 - __clz(max(lpk, 1));
    const size_t page_elems = (size_t)G * D * page_size;
    for (int ti = i_lo; ti < i_hi; ++ti) {
        const bool first = ti < tiles.n_a;
        const int jt = first ? ti * MA_TK : tiles.jt_b + (ti - tiles.n_a) * MA_TK;
        const int r_lo = first ? 0 : tiles.lo, r_hi = first ? tiles.a_hi : tiles.hi;
        int* chunk = chunk_s + (ti & 1) * (MA_TK / 4);
        if (tid < MA_TK / 8) {
            const int j = jt + tid * 8;
            chunk[tid] = j < r_hi ? table[j / page_size] : 0;       // (no page is looked up past the token's own)
            chunk[MA_TK / 8 + tid] = j % page_size;
        }
        // products of all heads' queries with the tile's keys
        if (rows_by_lanes) {
            const int kpi = 64 >> lpk_shift;           // keys a wave takes at a time
            const int kl = lane >> lpk_shift, dl = lane & (lpk - 1);
            const int its = G << lpk_shift;            // (MA_TK / kpi = lpk rounds a kv head)
            for (int it0 = wv; it0 < its; it0 += MA_WAVES * MA_AHEAD) {
                MaRaw<TC> rows[MA_AHEAD];
#pragma unroll
                for (int a = 0; a < MA_AHEAD; ++a) {
                    const int it = it0 + a * MA_WAVES;
                    const int kvh = it >> lpk_shift, j = jt + (it & (lpk - 1)) * kpi + kl;
                    rows[a].zero();
                    if (it < its && j >= r_lo && j < r_hi) {
                        const int page = table[j / page_size], off = j % page_size;
                        rows[a].load(k_cache + (((size_t)page * G + kvh) * page_size + off) * D + dl * 8);
                    }
                }
#pragma unroll
                for (int a = 0; a < MA_AHEAD; ++a) {
                    const int it = it0 + a * MA_WAVES;
                    if (it >= its) break;
                    const int kvh = it >> lpk_shift, key = (it & (lpk - 1)) * kpi + kl;
                    float kf[8];
                    rows[a].get(kf);
                    for (int g = kvh * rep; g < (kvh + 1) * rep; ++g) {
                        const float4* q4 = reinterpret_cast<const float4*>(q_s + g * D + dl * 8);
                        const float4 qa = q4[0], qb = q4[1];
                        float dot = qa.x * kf[0];
                        dot = fmaf(qa.y, kf[1], dot); dot = fmaf(qa.z, kf[2], dot); dot = fmaf(qa.w, kf[3], dot);
                        dot = fmaf(qb.x, kf[4], dot); dot = fmaf(qb.y, kf[5], dot); dot = fmaf(qb.z, kf[6], dot);
                        dot = fmaf(qb.w, kf[7], dot);
                        for (int o = 1; o < lpk; o <<= 1) dot += __shfl_xor(dot, o, 64);
                        if (dl == 0) s_raw[g * MA_TK + key] = dot;
                    }
                }
            }
        } else {
            const int j = jt + lane;
            const bool vis = j >= r_lo && j < r_hi;
            if (vis) {
                const int page = table[j / page_size], off = j % page_size;
                for (int g = wv; g < H; g += MA_WAVES) {
                    const TC* kr = k_cache + (((size_t)page * G + g / rep) * page_size + off) * D;
                    const float* qg = q_s + g * D;
                    float dot = 0.f;
                    for (int d = 0; d < D; ++d) dot = fmaf(qg[d], to_f32(kr[d]), dot);
                    s_raw[g * MA_TK + lane] = dot;
                }
            } else {
                for (int g = wv; g < H; g += MA_WAVES) s_raw[g * MA_TK + lane] = 0.f;
            }
        }
        __syncthreads();
        // scale, soft cap and the bias of the distance: a lane a key, a wave a head at a time
        {
            const int j = jt + lane;
            const bool vis = j >= r_lo && j < r_hi;
            const int dist = min(pos - j, bias_rows - 1);
            for (int g = wv; g < H; g += MA_WAVES) {
                float sc = 0.f;
                if (vis) {
                    sc = s_raw[g * MA_TK + lane] * scale;
                    if (cap > 0.f) sc = cap * tanhf(sc / cap);
                    if (bias) sc += bias[(size_t)dist * H + g];
                }
                s_raw[g * MA_TK + lane] = sc;
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
        // weighted values: thread -> (head, element) pairs; the tile's runs of 8 keys are asked for four at a time
        {
            const int c_lo = (max(jt, r_lo) - jt) >> 3, c_hi = (min(jt + MA_TK, r_hi) - jt + 7) >> 3;
#pragma unroll
            for (int n = 0; n < ACC; ++n) {
                const int idx = tid + n * MA_THREADS;
                if (idx < HD) {
                    const int h = idx / D;
                    const int voff = ((h / rep) * D + idx % D) * page_size;      // (kv head, element) in a value page
                    float a = acc[n] * c_s[h];
                    const float* ph = p_s + h * MA_TK;
#pragma unroll
                    for (int c0 = 0; c0 < MA_TK / 8; c0 += MA_RUNS) {
                        MaRaw<TC> runs[MA_RUNS];
#pragma unroll
                        for (int c = 0; c < MA_RUNS; ++c) {
                            runs[c].zero();
                            if (c0 + c >= c_lo && c0 + c < c_hi)        // (pages hold a multiple of 8 tokens)
                                runs[c].load(v_cache + (size_t)chunk[c0 + c] * page_elems + chunk[MA_TK / 8 + c0 + c] + voff);
                        }
#pragma unroll
                        for (int c = 0; c < MA_RUNS; ++c) {
                            float vf[8];
                            runs[c].get(vf);
#pragma unroll
                            for (int i = 0; i < 8; ++i) a = fmaf(ph[(c0 + c) * 8 + i], vf[i], a);
                        }
                    }
                    acc[n] = a;
                }
            }
        }
        // (the next tile's scores go to s_raw, which nobody reads any more; its barrier stands
        // between these reads of p_s and the next writes)
    }
    __syncthreads();
    if (nsplit == 1) {
#pragma unroll
        for (int n = 0; n < ACC; ++n) {
            const int idx = tid + n * MA_THREADS;
            if (idx < HD) {
                const float l = l_s[idx / D];
                out[(size_t)t * HD + idx] = from_f32<TC>(l > 0.f ? acc[n] / l : 0.f);
            }
        }
        return;
    }
    float* po = part_o + ((size_t)t * nsplit + split) * HD;
#pragma unroll
    for (int n = 0; n < ACC; ++n) {
        const int idx = tid + n * MA_THREADS;
        if (idx < HD) po[idx] = acc[n];
    }
    float* pm = part_ml + ((size_t)t * nsplit + split) * 2 * H;
    for (int i = tid; i < H; i += MA_THREADS) {
        pm[i] = m_s[i];
        pm[H + i] = l_s[i];
    }
}

// The splits of a token's keys put together, in the order of the splits: M = max of the maxima (and 0, the
// sink's score), L = [sink] e^-M + sum_s l_s e^(m_s - M), out = sum_s o_s e^(m_s - M) / L.
template <typename TC>
__global__ __launch_bounds__(64) void mixed_attention_merge_kernel(const float* __restrict__ part_o,
                                                                   const float* __restrict__ part_ml, int nsplit,
                                                                   int sink, TC* __restrict__ out, int H, int D) {
    const int t = blockIdx.x / H, h = blockIdx.x % H, HD = H * D;
    const float* pm = part_ml + (size_t)t * nsplit * 2 * H;
    const float* po = part_o + (size_t)t * nsplit * HD + (size_t)h * D;
    float M = sink ? 0.f : -INFINITY;
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, pm[s * 2 * H + h]);
    float L = sink ? expf(-M) : 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float m = pm[s * 2 * H + h];
        if (m > -INFINITY) L = fmaf(pm[s * 2 * H + H + h], expf(m - M), L);
    }
    for (int e = threadIdx.x; e < D; e += 64) {
        float a = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float m = pm[s * 2 * H + h];
            if (m > -INFINITY) a = fmaf(po[(size_t)s * HD + e], expf(m - M), a);
        }
        out[(size_t)t * HD + (size_t)h * D + e] = from_f32<TC>(L > 0.f ? a / L : 0.f);
    }
}

// ---- prompts in bfloat16: sixteen queries a block, the two products on the matrix cores ----
//
// A block takes up to 16 consecutive tokens of one request (a work item: first token, count) and all heads.
// Per tile of 16 keys (borders at multiples of 16 from the sequence's start):
//   1. S_g = Q_g K^T per head g: MFMA 16x16x32 over the head's elements, a wave a head at a time, operands straight
//      from memory (lane (row, quarter) holds 8 consecutive elements of its row); scale, cap and bias on the
//      accumulators; the scores go to LDS as float32 [head][query][key].
//   2. A thread per (head, query): the scores of all heads mixed, the mask, the running maximum and sum, the
//      weights to LDS as bfloat16 [head][query][key].
//   3. O_h += P_h V: MFMA 16x16x32 whose upper sixteen contraction slots are zero; values from the transposed
//      pages (a tile lies in one page: pages of a multiple of 16 tokens).
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 ma_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float ma_floatx4;

#define Q16_THREADS 512
#define Q16_WAVES 8
#define Q16_SROW 16      // floats a (head, query) row of scores takes in LDS
// Where key chunk c (four keys) of query qq lies in its row: rows lie 64 bytes apart, so without this the rows of
// every other query would meet in the same banks when sixteen threads read their own query's chunk c.
#define Q16_CHUNK(c, qq) (((c) ^ (((qq) >> 1) & 3)) * 4)

template <int HPW, int EB>
__global__ __launch_bounds__(Q16_THREADS) void mixed_attention_q16_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    const int32_t* __restrict__ block_tables, int bt_width, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ work, const float* __restrict__ bias,
    int bias_rows, const float* __restrict__ mix, float scale, float cap, int window, int keep_first, int sink,
    bf16_t* __restrict__ out, int H, int G, int page_size, int tiles_per_split, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
    constexpr int D = EB * 16, KC = D / 32;
    extern __shared__ float lds[];
    float* s_raw = lds;                                  // [H][16][Q16_SROW]
    float* mix_s = s_raw + H * 16 * Q16_SROW;            // [H][H] (if mix)
    float* m_s = mix_s + (mix ? (H * H + 3) / 4 * 4 : 0);  // [H][16] (16-byte aligned, as all that follows)
    float* l_s = m_s + H * 16;
    float* c_s = l_s + H * 16;
    bf16_t* p_s = reinterpret_cast<bf16_t*>(c_s + H * 16);   // [H][16][16]
    const int t0 = work[2 * blockIdx.x], n = work[2 * blockIdx.x + 1];
    const int split = blockIdx.y, nsplit = gridDim.y;
    const bool own_sink = sink && nsplit == 1;       // (with several splits the merge adds the sink's term)
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, col = lane & 15, g4 = lane >> 4;
    const int pos0 = positions[t0], pos_last = pos0 + n - 1;
    const int32_t* table = block_tables + (size_t)token_req[t0] * bt_width;
    const int rep = H / G, HD = H * D;
    if (mix)
        for (int i = tid; i < H * H; i += Q16_THREADS) mix_s[i] = mix[i];
    for (int i = tid; i < H * 16; i += Q16_THREADS) {
        m_s[i] = own_sink ? 0.f : -INFINITY;
        l_s[i] = own_sink ? 1.f : 0.f;
    }
    ma_floatx4 oacc[HPW][EB];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
        for (int eb = 0; eb < EB; ++eb) oacc[hh][eb] = ma_floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16_t* qrow = q + (size_t)(t0 + min(col, n - 1)) * HD + g4 * 8;
    const size_t page_elems = (size_t)G * D * page_size;
    __syncthreads();

    auto tile = [&](int jt) {
        // 1. scores: the wave's heads lie side by side, so they mostly share a kv head and its keys are fetched once;
        // all of a tile's operands are asked for before the first product
        {
            const int j = min(jt + col, pos_last);
            const bf16_t* kpage = k_cache + (size_t)table[j / page_size] * page_elems + (size_t)(j % page_size) * D + g4 * 8;
            // (the queries of all the wave's heads at once where the registers hold them beside the results)
            constexpr bool Q_AHEAD = HPW * KC <= 8;
            ma_bf16x8 qf[Q_AHEAD ? HPW : 1][KC], kf[KC];
            if (Q_AHEAD) {
#pragma unroll
                for (int hh = 0; hh < HPW; ++hh) {
                    const int h = min(wv * HPW + hh, H - 1);
#pragma unroll
                    for (int kc = 0; kc < KC; ++kc) qf[Q_AHEAD ? hh : 0][kc] = *reinterpret_cast<const ma_bf16x8*>(qrow + h * D + kc * 32);
                }
            }
            int kv_have = -1;
#pragma unroll
            for (int hh = 0; hh < HPW; ++hh) {
                const int h = wv * HPW + hh;
                if (h < H) {
                    if (h / rep != kv_have) {
                        kv_have = h / rep;
                        const bf16_t* krow = kpage + (size_t)kv_have * page_size * D;
#pragma unroll
                        for (int kc = 0; kc < KC; ++kc) kf[kc] = *reinterpret_cast<const ma_bf16x8*>(krow + kc * 32);
                    }
                    if (!Q_AHEAD) {
#pragma unroll
                        for (int kc = 0; kc < KC; ++kc) qf[0][kc] = *reinterpret_cast<const ma_bf16x8*>(qrow + h * D + kc * 32);
                    }
                    ma_floatx4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int kc = 0; kc < KC; ++kc)
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(qf[Q_AHEAD ? hh : 0][kc], kf[kc], acc, 0, 0, 0);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {        // (query g4 * 4 + i, key col)
                        const int qq = g4 * 4 + i;
                        float sc = acc[i] * scale;
                        if (cap > 0.f) sc = cap * tanhf(sc / cap);
                        if (bias) sc += bias[(size_t)min(max(pos0 + qq - (jt + col), 0), bias_rows - 1) * H + h];
                        s_raw[(h * 16 + qq) * Q16_SROW + Q16_CHUNK(col >> 2, qq) + (col & 3)] = sc;
                    }
                }
            }
        }
        __syncthreads();
        // 2. a thread per (head, query)
        {
            const int h = tid >> 4, qq = tid & 15;
            if (h < H) {
                float sm[16];
                if (mix) {
#pragma unroll
                    for (int kk = 0; kk < 16; ++kk) sm[kk] = 0.f;
                    for (int g = 0; g < H; ++g) {
                        const float tg = mix_s[h * H + g];
                        const float4* row = reinterpret_cast<const float4*>(s_raw + (g * 16 + qq) * Q16_SROW);
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            const float4 v4 = row[Q16_CHUNK(c, qq) >> 2];
                            sm[4 * c] = fmaf(tg, v4.x, sm[4 * c]);
                            sm[4 * c + 1] = fmaf(tg, v4.y, sm[4 * c + 1]);
                            sm[4 * c + 2] = fmaf(tg, v4.z, sm[4 * c + 2]);
                            sm[4 * c + 3] = fmaf(tg, v4.w, sm[4 * c + 3]);
                        }
                    }
                } else {
                    const float4* row = reinterpret_cast<const float4*>(s_raw + (h * 16 + qq) * Q16_SROW);
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const float4 v4 = row[Q16_CHUNK(c, qq) >> 2];
                        sm[4 * c] = v4.x; sm[4 * c + 1] = v4.y; sm[4 * c + 2] = v4.z; sm[4 * c + 3] = v4.w;
                    }
                }
                const int posq = pos0 + qq;
                const float m_old = m_s[h * 16 + qq];
                float mx = m_old;
                bool vis[16];
#pragma unroll
                for (int kk = 0; kk < 16; ++kk) {
                    const int j = jt + kk;
                    vis[kk] = qq < n && j <= posq && (window <= 0 || posq - j < window || j < keep_first);
                    if (vis[kk]) mx = fmaxf(mx, sm[kk]);
                }
                float corr = 1.f, sum = 0.f;
                if (mx > -INFINITY) corr = expf(m_old - mx);
                union { bf16_t h[16]; uint4 u[2]; } pk;
#pragma unroll
                for (int kk = 0; kk < 16; ++kk) {
                    // (the sum takes the weights as the product will see them)
                    const bf16_t pb = (bf16_t)(vis[kk] ? expf(sm[kk] - mx) : 0.f);
                    pk.h[kk] = pb;
                    sum += (float)pb;
                }
                m_s[h * 16 + qq] = mx;
                l_s[h * 16 + qq] = l_s[h * 16 + qq] * corr + sum;
                c_s[h * 16 + qq] = corr;
                uint4* pd = reinterpret_cast<uint4*>(p_s + (h * 16 + qq) * 16);
                pd[0] = pk.u[0];
                pd[1] = pk.u[1];
            }
        }
        __syncthreads();
        // 3. weighted values; where the wave's heads share a kv head its values are fetched once for all of them
        {
            const bf16_t* vpage = v_cache + (size_t)table[jt / page_size] * page_elems + (size_t)col * page_size + jt % page_size + g4 * 8;
            const ma_bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
            const int h_lo = wv * HPW, h_hi = min(h_lo + HPW, H) - 1;
            const bool one_kv = h_lo < H && h_lo / rep == h_hi / rep;
            constexpr int VG = HPW * EB >= 32 ? 2 : (EB < 4 ? EB : 4);      // value fragments asked for at a time (fewer where the results fill the registers)
#pragma unroll
            for (int e0 = 0; e0 < EB; e0 += VG) {
                ma_bf16x8 vb[VG];
                if (one_kv) {
                    const bf16_t* vhead = vpage + (size_t)(h_lo / rep) * D * page_size;
#pragma unroll
                    for (int e = 0; e < VG; ++e)
                        vb[e] = g4 < 2 ? *reinterpret_cast<const ma_bf16x8*>(vhead + (size_t)(e0 + e) * 16 * page_size) : zero;
                }
#pragma unroll
                for (int hh = 0; hh < HPW; ++hh) {
                    const int h = h_lo + hh;
                    if (h < H) {
                        const bf16_t* vhead = vpage + (size_t)(h / rep) * D * page_size;
                        // (the head's weights and factors come from LDS again for every group: registers are dearer)
                        const ma_bf16x8 pa = g4 < 2 ? *reinterpret_cast<const ma_bf16x8*>(p_s + (h * 16 + col) * 16 + g4 * 8) : zero;
                        float cr[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) cr[i] = c_s[h * 16 + g4 * 4 + i];
#pragma unroll
                        for (int e = 0; e < VG; ++e) {
                            const ma_bf16x8 b = one_kv ? vb[e]
                                                       : (g4 < 2 ? *reinterpret_cast<const ma_bf16x8*>(vhead + (size_t)(e0 + e) * 16 * page_size) : zero);
#pragma unroll
                            for (int i = 0; i < 4; ++i) oacc[hh][e0 + e][i] *= cr[i];
                            oacc[hh][e0 + e] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pa, b, oacc[hh][e0 + e], 0, 0, 0);
                        }
                    }
                }
            }
        }
        // (the next tile's scores go to s_raw, which nobody reads any more; its first barrier stands between these
        // reads of p_s and c_s and their next writes)
    };

    const int lo_first = window > 0 ? max(0, pos0 - window + 1) : 0;
    const int lo_last = window > 0 ? max(0, pos_last - window + 1) : 0;
    const int jt_b = (lo_first / 16) * 16;
    // the block's tiles, numbered through: those of the kept first tokens before the windows, then the windows'
    const int n_a = (min(min(keep_first, lo_last), jt_b) + 15) / 16;
    const int tiles = n_a + (pos_last - jt_b) / 16 + 1;
    const int i_lo = nsplit == 1 ? 0 : split * tiles_per_split;
    const int i_hi = split == nsplit - 1 ? tiles : min(tiles, i_lo + tiles_per_split);      // (the last split takes what is left)
    for (int ti = i_lo; ti < i_hi; ++ti) tile(ti < n_a ? ti * 16 : jt_b + (ti - n_a) * 16);
    __syncthreads();
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        const int h = wv * HPW + hh;
        if (h < H) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int qq = g4 * 4 + i;
                if (qq < n) {
                    if (nsplit == 1) {
                        const float l = l_s[h * 16 + qq];
                        const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
                        for (int eb = 0; eb < EB; ++eb)
                            out[(size_t)(t0 + qq) * HD + h * D + eb * 16 + col] = (bf16_t)(oacc[hh][eb][i] * inv);
                    } else {
                        float* po = part_o + ((size_t)(t0 + qq) * nsplit + split) * HD + h * D + col;
#pragma unroll
                        for (int eb = 0; eb < EB; ++eb) po[eb * 16] = oacc[hh][eb][i];
                    }
                }
            }
        }
    }
    if (nsplit > 1) {
        // (maximum and sum per head and query, in the merge's layout: [token][split][maxima of the heads | sums])
        const int h = tid >> 4, qq = tid & 15;
        if (h < H && qq < n) {
            float* pm = part_ml + ((size_t)(t0 + qq) * nsplit + split) * 2 * H;
            pm[h] = m_s[h * 16 + qq];
            pm[H + h] = l_s[h * 16 + qq];
        }
    }
}

static size_t q16_lds_bytes(int H, bool mix) {
    return sizeof(float) * ((size_t)H * 16 * Q16_SROW + (mix ? ((size_t)H * H + 3) / 4 * 4 : 0) + 3 * (size_t)H * 16) + 2 * (size_t)H * 256;
}

// bfloat16, up to 32 heads of 32, 64 or 128 elements, pages of a multiple of 16 tokens.
TFF_API int tff_mixed_attention_q16_supported(int H, int D, int page_size, int has_mix) {
    return H > 0 && H <= 32 && (D == 32 || D == 64 || D == 128) && page_size % 16 == 0 &&
           q16_lds_bytes(H, has_mix != 0) <= 64 * 1024;
}

// work: int32 [items][2] = (first token of the step, count <= 16), the tokens of an item consecutive tokens of one
// request; every one of the step's T tokens lies in one item.  splits > 1: an item's tiles of 16 keys are dealt to
// `splits` blocks, tiles_per_split each, and merged as tff_mixed_attention's are (the same workspace size).
TFF_API int tff_mixed_attention_q16(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                    int bt_width, const int32_t* token_req, const int32_t* positions, const int32_t* work,
                                    int items, const float* bias, int bias_rows, const float* mix, float scale, float cap,
                                    int window, int keep_first, int sink, void* out, int T, int H, int G, int D,
                                    int page_size, int splits, int tiles_per_split, float* workspace, tff_stream_t stream) {
    TFF_REQUIRE(q && k_cache && v_cache && block_tables && token_req && positions && work && out,
                "mixed_attention_q16: null pointer");
    TFF_REQUIRE(splits >= 1 && splits <= 65535 && (splits == 1 || (tiles_per_split >= 1 && workspace)),
                "mixed_attention_q16: %d splits of %d tiles", splits, tiles_per_split);
    TFF_REQUIRE(G > 0 && H % G == 0 && bt_width > 0 && tff_mixed_attention_q16_supported(H, D, page_size, mix != nullptr),
                "mixed_attention_q16: %d heads of %d on %d kv heads, pages of %d", H, D, G, page_size);
    TFF_REQUIRE(!bias || bias_rows > 0, "mixed_attention_q16: a bias table without rows");
    TFF_REQUIRE(window >= 0 && keep_first >= 0 && items >= 0, "mixed_attention_q16: negative sizes");
    if (items == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = q16_lds_bytes(H, mix != nullptr);
    const int hpw = (H + Q16_WAVES - 1) / Q16_WAVES;
    float* part_o = workspace;
    float* part_ml = workspace ? workspace + (size_t)T * splits * H * D : nullptr;
#define Q16_LAUNCH(HPW, EB)                                                                                          \
    mixed_attention_q16_kernel<HPW, EB><<<dim3(items, splits), Q16_THREADS, lds, s>>>(                              \
        (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, bt_width, token_req,       \
        positions, work, bias, bias_rows, mix, scale, cap, window, keep_first, sink, (bf16_t*)out, H, G, page_size, \
        tiles_per_split, part_o, part_ml)
#define Q16_BY_EB(HPW)                  \
    do {                                \
        if (D == 32) Q16_LAUNCH(HPW, 2); \
        else if (D == 64) Q16_LAUNCH(HPW, 4); \
        else Q16_LAUNCH(HPW, 8);        \
    } while (0)
    if (hpw <= 1) Q16_BY_EB(1);
    else if (hpw <= 2) Q16_BY_EB(2);
    else Q16_BY_EB(4);
#undef Q16_BY_EB
#undef Q16_LAUNCH
    int rc = tff_check_launch("mixed_attention_q16");
    if (rc || splits <= 1) return rc;
    mixed_attention_merge_kernel<bf16_t><<<T * H, 64, 0, s>>>(part_o, part_ml, splits, sink, (bf16_t*)out, H, D);
    return tff_check_launch("mixed_attention_merge");
}

static size_t ma_lds_bytes(int H, int D, bool mix) {
    return sizeof(float) * ((size_t)H * D + 2 * (size_t)H * MA_TK + (mix ? (size_t)H * H : 0) + 3 * (size_t)H + MA_TK / 2);
}

TFF_API int tff_mixed_attention_supported(int H, int D, int has_mix) {
    return H > 0 && D > 0 && (size_t)H * D <= 8 * MA_THREADS && ma_lds_bytes(H, D, has_mix != 0) <= 64 * 1024;
}

// Floats of workspace that `splits` splits of T tokens need (0 for one split).
TFF_API size_t tff_mixed_attention_workspace_bytes(int T, int H, int D, int splits) {
    return splits <= 1 ? 0 : sizeof(float) * (size_t)T * splits * ((size_t)H * D + 2 * (size_t)H);
}

template <typename TC>
static int ma_launch(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables, int bt_width,
                     const int32_t* token_req, const int32_t* positions, const float* bias, int bias_rows, const float* mix,
                     float scale, float cap, int window, int keep_first, int sink, void* out, int T, int H, int G, int D,
                     int page_size, int splits, int tiles_per_split, float* ws, hipStream_t s) {
    const size_t lds = ma_lds_bytes(H, D, mix != nullptr);
    const int per = (H * D + MA_THREADS - 1) / MA_THREADS;
    float* part_o = ws;
    float* part_ml = ws ? ws + (size_t)T * splits * H * D : nullptr;
    const dim3 grid(T, splits);
#define MA_LAUNCH(ACC)                                                                                                   \
    mixed_attention_kernel<TC, ACC><<<grid, MA_THREADS, lds, s>>>((const TC*)q, (const TC*)k_cache, (const TC*)v_cache,   \
                                                                   block_tables, bt_width, token_req, positions, bias,   \
                                                                   bias_rows, mix, scale, cap, window, keep_first, sink, \
                                                                   (TC*)out, H, G, D, page_size, tiles_per_split, part_o, \
                                                                   part_ml)
    if (per <= 1) MA_LAUNCH(1);
    else if (per <= 2) MA_LAUNCH(2);
    else if (per <= 4) MA_LAUNCH(4);
    else MA_LAUNCH(8);
#undef MA_LAUNCH
    int rc = tff_check_launch("mixed_attention");
    if (rc || splits <= 1) return rc;
    mixed_attention_merge_kernel<TC><<<T * H, 64, 0, s>>>(part_o, part_ml, splits, sink, (TC*)out, H, D);
    return tff_check_launch("mixed_attention_merge");
}

TFF_API int tff_mixed_attention(const void* q, const void* k_cache, const void* v_cache, const int32_t* block_tables,
                                int bt_width, const int32_t* token_req, const int32_t* positions, const float* bias,
                                int bias_rows, const float* mix, float scale, float cap, int window, int keep_first,
                                int sink, void* out, int T, int H, int G, int D, int page_size, int splits,
                                int tiles_per_split, float* workspace, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(q && k_cache && v_cache && block_tables && token_req && positions && out, "mixed_attention: null pointer");
    TFF_REQUIRE(T >= 0 && G > 0 && H % G == 0 && bt_width > 0 && page_size > 0 && page_size % 8 == 0,
                "mixed_attention: %d heads on %d kv heads, pages of %d", H, G, page_size);
    TFF_REQUIRE(tff_mixed_attention_supported(H, D, mix != nullptr), "mixed_attention: %d heads of %d do not fit a block", H, D);
    TFF_REQUIRE(!bias || bias_rows > 0, "mixed_attention: a bias table without rows");
    TFF_REQUIRE(window >= 0 && keep_first >= 0, "mixed_attention: negative window");
    TFF_REQUIRE(splits >= 1 && splits <= 65535 && (splits == 1 || (tiles_per_split >= 1 && workspace)),
                "mixed_attention: %d splits of %d tiles", splits, tiles_per_split);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        return ma_launch<float>(q, k_cache, v_cache, block_tables, bt_width, token_req, positions, bias, bias_rows, mix,
                                scale, cap, window, keep_first, sink, out, T, H, G, D, page_size, splits, tiles_per_split,
                                workspace, s);
    if (dtype == TFF_BF16)
        return ma_launch<bf16_t>(q, k_cache, v_cache, block_tables, bt_width, token_req, positions, bias, bias_rows, mix,
                                 scale, cap, window, keep_first, sink, out, T, H, G, D, page_size, splits, tiles_per_split,
                                 workspace, s);
    return tff_fail("mixed_attention: unknown dtype %d", dtype);
}
