// A linear recurrence with a matrix of state per head (time mixing in the manner of RWKV):
//
//   o_t = (S_{t-1} + diag(u) k_t v_t^T)^T r_t,      S_t = diag(w_t) S_{t-1} + k_t v_t^T,
//   w_t = exp(-exp(z_t + w0))                        (per head and key channel, float32)
//
// with S [key channel, value channel] per request and head in float32, carried from step to
// step in the request's state row.  The inputs of the projections are mixes of a token's row
// with the row of the token before it, whose last one is part of the state as well.
//
// tff_token_shift_mix: out[m, t, :] = x[t] + (x'[t] - x[t]) * mu[m], x' the row of the token
//   before t in the same request: the row above, or for the first token of a request's portion
//   the row that the state keeps (zeros for a request's first token).
// tff_wkv_recurrence: the recurrence over the tokens of each request's portion, one block per
//   (head, request), a thread per value channel and slice of the key channels; the order of every
//   sum is fixed by the head size alone, so a token's result does not depend on how the tokens
//   were cut into steps.  The block of head 0 also leaves the portion's last row of x in the state.
// tff_head_norm_gate: out = o / sqrt(mean over the head of o^2 + eps) * weight * silu(g).
// tff_tanh: out = tanh(in), float32 in, the activation type out.
#include "common.h"
#include "tffinfer_kernels.h"

template <typename TO>
__global__ __launch_bounds__(256) void token_shift_mix_kernel(
    const float* __restrict__ x, const float* __restrict__ state, size_t state_row, size_t prev_off,
    const float* __restrict__ mu, int M, const int32_t* __restrict__ token_req,
    const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ state_slots, TO* __restrict__ out, int T,
    int W) {
    const int t = blockIdx.x;
    const int r = token_req[t];
    const float* prev = (t == cu_tokens[r]) ? state + (size_t)state_slots[r] * state_row + prev_off
                                            : x + (size_t)(t - 1) * W;
    const float* xr = x + (size_t)t * W;
    for (int c = threadIdx.x; c < W; c += 256) {
        const float h = xr[c];
        const float d = prev[c] - h;
        for (int m = 0; m < M; ++m) out[((size_t)m * T + t) * W + c] = from_f32<TO>(h + d * mu[(size_t)m * W + c]);
    }
}

TFF_API int tff_token_shift_mix(const float* x, const float* state, size_t state_row, size_t prev_off, const float* mu,
                                int M, const int32_t* token_req, const int32_t* cu_tokens, const int32_t* state_slots,
                                void* out, int T, int W, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(x && state && mu && token_req && cu_tokens && state_slots && out, "token_shift_mix: null pointer");
    TFF_REQUIRE(T >= 0 && W > 0 && M > 0 && prev_off + (size_t)W <= state_row, "token_shift_mix: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (out_dtype == TFF_F32)
        token_shift_mix_kernel<float><<<T, 256, 0, s>>>(x, state, state_row, prev_off, mu, M, token_req, cu_tokens,
                                                         state_slots, (float*)out, T, W);
    else if (out_dtype == TFF_BF16)
        token_shift_mix_kernel<bf16_t><<<T, 256, 0, s>>>(x, state, state_row, prev_off, mu, M, token_req, cu_tokens,
                                                          state_slots, (bf16_t*)out, T, W);
    else
        return tff_fail("token_shift_mix: unknown dtype %d", out_dtype);
    return tff_check_launch("token_shift_mix");
}

#define WKV_MAX_D 128     // (a thread keeps a slice of a column of S in registers)
#define WKV_MAX_SLICES 4

// KPT key channels a thread; ceil(D / KPT) <= 4 slices of the key channels; thread = slice * D + value channel.
template <int KPT>
__global__ __launch_bounds__(512) void wkv_recurrence_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ z, size_t row, const float* __restrict__ w0, const float* __restrict__ u,
    float* __restrict__ state, size_t state_row, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ state_slots, float* __restrict__ o, int H, int D, const float* __restrict__ x, int W,
    size_t prev_off) {
    __shared__ float sr[2][WKV_MAX_D], sk[2][WKV_MAX_D], sw[2][WKV_MAX_D], su[WKV_MAX_D];
    __shared__ float part[WKV_MAX_SLICES][WKV_MAX_D];
    const int h = blockIdx.x, req = blockIdx.y, tid = threadIdx.x;
    const int t0 = cu_tokens[req], t1 = cu_tokens[req + 1];
    if (t1 <= t0) return;
    const int slices = blockDim.x / D;
    const int vi = tid % D, ks = tid / D;
    float* srow = state + (size_t)state_slots[req] * state_row;
    float* S = srow + (size_t)h * D * D;
    const size_t col = (size_t)h * D;
    float s[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int kk = ks * KPT + i;
        s[i] = kk < D ? S[(size_t)kk * D + vi] : 0.f;
    }
    if (tid < D) {
        su[tid] = u[col + tid];
        const size_t a = (size_t)t0 * row + col + tid;
        sr[0][tid] = r[a];
        sk[0][tid] = k[a];
        sw[0][tid] = expf(-expf(z[a] + w0[col + tid]));
    }
    for (int t = t0; t < t1; ++t) {
        const int b = (t - t0) & 1;
        __syncthreads();
        const float vt = v[(size_t)t * row + col + vi];
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < KPT; ++i) {
            const int kk = ks * KPT + i;
            if (kk < D) {
                const float kv = sk[b][kk] * vt;
                acc = fmaf(sr[b][kk], fmaf(su[kk], kv, s[i]), acc);
                s[i] = fmaf(sw[b][kk], s[i], kv);
            }
        }
        part[ks][vi] = acc;
        if (t + 1 < t1 && tid < D) {
            const size_t a = (size_t)(t + 1) * row + col + tid;
            sr[b ^ 1][tid] = r[a];
            sk[b ^ 1][tid] = k[a];
            sw[b ^ 1][tid] = expf(-expf(z[a] + w0[col + tid]));
        }
        __syncthreads();
        if (ks == 0) {
            float sum = part[0][vi];
            for (int p = 1; p < slices; ++p) sum += part[p][vi];
            o[(size_t)t * H * D + col + vi] = sum;
        }
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int kk = ks * KPT + i;
        if (kk < D) S[(size_t)kk * D + vi] = s[i];
    }
    if (h == 0 && x) {
        const float* last = x + (size_t)(t1 - 1) * W;
        for (int c = tid; c < W; c += blockDim.x) srow[prev_off + c] = last[c];
    }
}

TFF_API int tff_wkv_recurrence(const float* r, const float* k, const float* v, const float* z, size_t row, const float* w0,
                               const float* u, float* state, size_t state_row, const int32_t* cu_tokens,
                               const int32_t* state_slots, float* o, int R, int H, int D, const float* x, int W,
                               size_t prev_off, tff_stream_t stream) {
    TFF_REQUIRE(r && k && v && z && w0 && u && state && cu_tokens && state_slots && o, "wkv_recurrence: null pointer");
    TFF_REQUIRE(R >= 0 && H > 0 && D > 0 && D <= WKV_MAX_D, "wkv_recurrence: %d heads of %d (up to %d)", H, D, WKV_MAX_D);
    TFF_REQUIRE(row >= (size_t)H * D && (size_t)H * D * D <= state_row && (!x || prev_off + (size_t)W <= state_row),
                "wkv_recurrence: rows of %zu, state rows of %zu do not hold %d heads of %d", row, state_row, H, D);
    if (R == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(H, R);
#define WKV_LAUNCH(KPT)                                                                                              \
    wkv_recurrence_kernel<KPT><<<grid, D * ((D + KPT - 1) / KPT), 0, s>>>(r, k, v, z, row, w0, u, state, state_row, \
                                                                           cu_tokens, state_slots, o, H, D, x, W, prev_off)
    if (D <= 64) WKV_LAUNCH(16);
    else WKV_LAUNCH(32);
#undef WKV_LAUNCH
    return tff_check_launch("wkv_recurrence");
}

template <typename TO>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ g,
                                                             size_t g_row, const float* __restrict__ nw, float eps,
                                                             TO* __restrict__ out, int pairs, int H, int D) {
    const int id = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (id >= pairs) return;
    const int t = id / H, h = id % H;
    const float* orow = o + ((size_t)t * H + h) * D;
    float ss = 0.f;
    for (int e = lane; e < D; e += 64) ss = fmaf(orow[e], orow[e], ss);
    ss = wave_sum(ss);
    const float rr = 1.0f / sqrtf(ss / (float)D + eps);
    const float* grow = g + (size_t)t * g_row + (size_t)h * D;
    for (int e = lane; e < D; e += 64) {
        const float gz = grow[e];
        const float gate = gz / (1.0f + expf(-gz));
        out[((size_t)t * H + h) * D + e] = from_f32<TO>(orow[e] * rr * nw[h * D + e] * gate);
    }
}

TFF_API int tff_head_norm_gate(const float* o, const float* g, size_t g_row, const float* nw, float eps, void* out, int T,
                               int H, int D, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(o && g && nw && out, "head_norm_gate: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && D > 0 && g_row >= (size_t)H * D, "head_norm_gate: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int pairs = T * H;
    if (out_dtype == TFF_F32)
        head_norm_gate_kernel<float><<<(pairs + 3) / 4, 256, 0, s>>>(o, g, g_row, nw, eps, (float*)out, pairs, H, D);
    else if (out_dtype == TFF_BF16)
        head_norm_gate_kernel<bf16_t><<<(pairs + 3) / 4, 256, 0, s>>>(o, g, g_row, nw, eps, (bf16_t*)out, pairs, H, D);
    else
        return tff_fail("head_norm_gate: unknown dtype %d", out_dtype);
    return tff_check_launch("head_norm_gate");
}

template <typename TO>
__global__ __launch_bounds__(256) void tanh_kernel(const float* __restrict__ in, TO* __restrict__ out, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) out[i] = from_f32<TO>(tanhf(in[i]));
}

TFF_API int tff_tanh(const float* in, void* out, size_t count, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(in && out, "tanh: null pointer");
    if (count == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (out_dtype == TFF_F32)
        tanh_kernel<float><<<blocks, 256, 0, s>>>(in, (float*)out, count);
    else if (out_dtype == TFF_BF16)
        tanh_kernel<bf16_t><<<blocks, 256, 0, s>>>(in, (bf16_t*)out, count);
    else
        return tff_fail("tanh: unknown dtype %d", out_dtype);
    return tff_check_launch("tanh");
}
