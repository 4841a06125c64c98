// The norm of a block that norms AFTER the residual sum:
//   v = alpha * x + delta;   x <- v / sqrt(mean(v^2) + eps) * w
// in place on the float32 residual stream, with a copy in the activation type for the products
// that read x next.  Sum, mean, root and products in float32.  delta may come as `planes`
// partial sums, `plane` elements apart, which are added up first, plane 0, 1, ... in turn
// (what tff_gemm leaves with keep_partials), or not at all (a layer without the sublayer).
//
// tff_gelu: the feed-forward's activation, exact (erf) or the tanh form, in float32.
#include "common.h"
#include "tffinfer_kernels.h"

#define PN_THREADS 256
#define PN_ITS 16      // rows of up to 4096 elements pass through memory once

template <typename TO>
__global__ __launch_bounds__(PN_THREADS) void scale_add_rmsnorm_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, int planes, size_t plane, float alpha,
    const float* __restrict__ w, float eps, TO* __restrict__ out, int H) {
    __shared__ float red[17];
    const int r = blockIdx.x, tid = threadIdx.x;
    float* x = resid + (size_t)r * H;
    const float* dl = delta ? delta + (size_t)r * H : nullptr;
    float cache[PN_ITS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < PN_ITS; ++it) {
        const int j = tid + it * PN_THREADS;
        if (j < H) {
            float v = alpha * x[j];
            if (dl) {
                float d = dl[j];
                for (int p = 1; p < planes; ++p) d += dl[p * plane + j];
                v += d;
            }
            cache[it] = v;
            ss = fmaf(v, v, ss);
        }
    }
    for (int j = tid + PN_ITS * PN_THREADS; j < H; j += PN_THREADS) {
        float v = alpha * x[j];
        if (dl) {
            float d = dl[j];
            for (int p = 1; p < planes; ++p) d += dl[p * plane + j];
            v += d;
        }
        x[j] = v;       // (kept in place for the second sweep)
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float rr = 1.0f / sqrtf(ss / (float)H + eps);
    TO* o = out ? out + (size_t)r * H : nullptr;
#pragma unroll
    for (int it = 0; it < PN_ITS; ++it) {
        const int j = tid + it * PN_THREADS;
        if (j < H) {
            const float y = cache[it] * rr * w[j];
            x[j] = y;
            if (o) o[j] = from_f32<TO>(y);
        }
    }
    for (int j = tid + PN_ITS * PN_THREADS; j < H; j += PN_THREADS) {
        const float y = x[j] * rr * w[j];
        x[j] = y;
        if (o) o[j] = from_f32<TO>(y);
    }
}

TFF_API int tff_scale_add_rmsnorm(float* resid, const float* delta, int delta_planes, size_t delta_plane, float alpha,
                                  const float* weight, float eps, void* out, int n, int H, int out_dtype,
                                  tff_stream_t stream) {
    TFF_REQUIRE(resid && weight, "scale_add_rmsnorm: null pointer");
    TFF_REQUIRE(n >= 0 && H > 0, "scale_add_rmsnorm: bad sizes n=%d H=%d", n, H);
    TFF_REQUIRE(!delta || delta_planes >= 1, "scale_add_rmsnorm: %d planes of partial sums", delta_planes);
    TFF_REQUIRE(out_dtype == TFF_F32 || out_dtype == TFF_BF16, "scale_add_rmsnorm: unknown dtype %d", out_dtype);
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int planes = delta ? delta_planes : 0;
    if (out_dtype == TFF_F32)
        scale_add_rmsnorm_kernel<float><<<n, PN_THREADS, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps,
                                                                 (float*)out, H);
    else
        scale_add_rmsnorm_kernel<bf16_t><<<n, PN_THREADS, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps,
                                                                  (bf16_t*)out, H);
    return tff_check_launch("scale_add_rmsnorm");
}

template <typename T>
__global__ void gelu_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t n, int tanh_form) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = to_f32(x[i]);
    float y;
    if (tanh_form)
        y = 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    else
        y = 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
    out[i] = from_f32<T>(y);
}

TFF_API int tff_gelu(const void* x, void* out, int64_t n, int tanh_form, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(x && out, "gelu: null pointer");
    TFF_REQUIRE(n >= 0, "gelu: negative size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == TFF_F32)
        gelu_kernel<float><<<blocks, 256, 0, s>>>((const float*)x, (float*)out, n, tanh_form);
    else if (dtype == TFF_BF16)
        gelu_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)x, (bf16_t*)out, n, tanh_form);
    else
        return tff_fail("gelu: unknown dtype %d", dtype);
    return tff_check_launch("gelu");
}
