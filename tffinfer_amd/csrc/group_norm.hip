// Norms on a sublayer's OUTPUT and sums over the depth of the model.
//
// tff_group_rmsnorm_add: a row of `delta` (a sublayer's output, perhaps as `planes` partial sums,
//   `plane` elements apart, added up first in their order) is cut into `groups` equal consecutive
//   parts; each part is divided by its own sqrt(mean(part^2) + eps); the whole is multiplied by w.
//   With `resid` the result is added into that row of the float32 residual stream, and `out`
//   (optional) gets the new row in the activation type.  Without `resid` the result itself goes to
//   `out`; `rows` (optional) then names the rows of `delta` to take (the rows whose logits are
//   wanted).  Sums, means, roots and products in float32.
// tff_depth_average: hist[n - 1] <- x;  x <- sum_{j < n} coef[j] * hist[j] (j ascending), with
//   hist [depths, T, W] the outputs of the embedding and of the layers so far; `out` (optional)
//   gets x in the activation type.
// tff_scale_rows: x <- alpha * x on float32 rows.
#include "common.h"
#include "tffinfer_kernels.h"

#define GN_THREADS 256

#define GN_ITS 8       // a group of up to 2048 elements passes through memory once

// One block per (row, group).
template <typename TO>
__global__ __launch_bounds__(GN_THREADS) void group_rmsnorm_add_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, int planes, size_t plane,
    const int32_t* __restrict__ rows, const float* __restrict__ w, int groups, float eps,
    TO* __restrict__ out, int H) {
    __shared__ float red[17];
    const int r = blockIdx.x / groups, g = blockIdx.x % groups, tid = threadIdx.x;
    const int src = rows ? rows[r] : r;
    const int Hg = H / groups, base = g * Hg;
    const float* dl = delta + (size_t)src * H + base;
    float* x = resid ? resid + (size_t)r * H + base : nullptr;
    TO* o = out ? out + (size_t)r * H + base : nullptr;
    const float* wg = w + base;
    auto term = [&](int j) {
        float d = dl[j];
        for (int p = 1; p < planes; ++p) d += dl[p * plane + j];
        return d;
    };
    float cache[GN_ITS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < GN_ITS; ++it) {
        const int j = tid + it * GN_THREADS;
        if (j < Hg) {
            cache[it] = term(j);
            ss = fmaf(cache[it], cache[it], ss);
        }
    }
    for (int j = tid + GN_ITS * GN_THREADS; j < Hg; j += GN_THREADS) {
        const float d = term(j);
        ss = fmaf(d, d, ss);
    }
    ss = block_sum(ss, red);
    const float rr = 1.0f / sqrtf(ss / (float)Hg + eps);
    auto emit = [&](int j, float d) {
        float y = d * rr * wg[j];
        if (x) {
            y += x[j];
            x[j] = y;
        }
        if (o) o[j] = from_f32<TO>(y);
    };
#pragma unroll
    for (int it = 0; it < GN_ITS; ++it) {
        const int j = tid + it * GN_THREADS;
        if (j < Hg) emit(j, cache[it]);
    }
    for (int j = tid + GN_ITS * GN_THREADS; j < Hg; j += GN_THREADS) emit(j, term(j));
}

TFF_API int tff_group_rmsnorm_add(float* resid, const float* delta, int planes, size_t plane, const int32_t* rows,
                                  const float* w, int groups, float eps, void* out, int n, int H, int out_dtype,
                                  tff_stream_t stream) {
    TFF_REQUIRE(delta && w && (resid || out), "group_rmsnorm_add: null pointer");
    TFF_REQUIRE(n >= 0 && H > 0 && groups > 0 && H % groups == 0, "group_rmsnorm_add: rows of %d in %d groups", H, groups);
    TFF_REQUIRE(planes >= 1 && !(rows && (resid || planes > 1)), "group_rmsnorm_add: bad combination of operands");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (!out || out_dtype == TFF_F32)
        group_rmsnorm_add_kernel<float><<<n * groups, GN_THREADS, 0, s>>>(resid, delta, planes, plane, rows, w, groups, eps,
                                                                  (float*)out, H);
    else if (out_dtype == TFF_BF16)
        group_rmsnorm_add_kernel<bf16_t><<<n * groups, GN_THREADS, 0, s>>>(resid, delta, planes, plane, rows, w, groups, eps,
                                                                   (bf16_t*)out, H);
    else
        return tff_fail("group_rmsnorm_add: unknown dtype %d", out_dtype);
    return tff_check_launch("group_rmsnorm_add");
}

template <typename TO>
__global__ __launch_bounds__(256) void depth_average_kernel(float* __restrict__ hist, size_t level, int n,
                                                            const float* __restrict__ coef, float* __restrict__ x,
                                                            TO* __restrict__ out, size_t count) {
    // four elements a thread; `count` is a multiple of 4 or the tail goes one by one
    const size_t i4 = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i4 >= count) return;
    const int m = (int)((count - i4) < 4 ? (count - i4) : 4);
    float v[4], acc[4];
    for (int e = 0; e < m; ++e) {
        v[e] = x[i4 + e];
        acc[e] = 0.f;
    }
    for (int j = 0; j + 1 < n; ++j) {
        const float c = coef[j];
        const float* hj = hist + (size_t)j * level + i4;
        for (int e = 0; e < m; ++e) acc[e] = fmaf(c, hj[e], acc[e]);
    }
    const float cl = coef[n - 1];
    float* hl = hist + (size_t)(n - 1) * level + i4;
    for (int e = 0; e < m; ++e) {
        hl[e] = v[e];
        const float y = fmaf(cl, v[e], acc[e]);
        x[i4 + e] = y;
        if (out) out[i4 + e] = from_f32<TO>(y);
    }
}

TFF_API int tff_depth_average(float* hist, size_t level, int n, const float* coef, float* x, void* out, size_t count,
                              int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(hist && coef && x, "depth_average: null pointer");
    TFF_REQUIRE(n >= 1 && level >= count, "depth_average: %d levels of %zu for %zu elements", n, level, count);
    if (count == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((count + 1023) / 1024);
    if (!out || out_dtype == TFF_F32)
        depth_average_kernel<float><<<blocks, 256, 0, s>>>(hist, level, n, coef, x, (float*)out, count);
    else if (out_dtype == TFF_BF16)
        depth_average_kernel<bf16_t><<<blocks, 256, 0, s>>>(hist, level, n, coef, x, (bf16_t*)out, count);
    else
        return tff_fail("depth_average: unknown dtype %d", out_dtype);
    return tff_check_launch("depth_average");
}

__global__ __launch_bounds__(256) void scale_rows_kernel(float* __restrict__ x, float alpha, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) x[i] *= alpha;
}

TFF_API int tff_scale_rows(float* x, float alpha, size_t count, tff_stream_t stream) {
    TFF_REQUIRE(x, "scale_rows: null pointer");
    if (count == 0) return 0;
    scale_rows_kernel<<<(unsigned)((count + 255) / 256), 256, 0, (hipStream_t)stream>>>(x, alpha, count);
    return tff_check_launch("scale_rows");
}
