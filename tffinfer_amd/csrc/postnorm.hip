// The norm of a block that norms AFTER the residual sum:
//   v = alpha * x + delta;   x <- v / sqrt(mean(v^2) + eps) * w
// in place on the float32 residual stream, with a copy in the activation type for the products
// that read x next.  Sum, mean, root and products in float32.  delta may come as `planes`
// partial sums, `plane` elements apart, which are added up first, plane 0, 1, ... in turn
// (what tff_gemm leaves with keep_partials), or not at all (a layer without the sublayer).
//
// tff_gelu: the feed-forward's activation, gelu exact (erf) or in the tanh form, or the square of relu, in float32.
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

// The same for rows whose width is a multiple of 4: 16-byte accesses; NT threads a row (1024 where
// there are few rows: more loads in flight for each), rows of up to 4096 elements in registers.
template <typename TO>
__device__ __forceinline__ void pn_store4(TO* o, float4 v);
template <>
__device__ __forceinline__ void pn_store4<float>(float* o, float4 v) { *reinterpret_cast<float4*>(o) = v; }
template <>
__device__ __forceinline__ void pn_store4<bf16_t>(bf16_t* o, float4 v) {
    union { bf16_t h[4]; uint2 u; } pk;
    pk.h[0] = (bf16_t)v.x; pk.h[1] = (bf16_t)v.y; pk.h[2] = (bf16_t)v.z; pk.h[3] = (bf16_t)v.w;
    *reinterpret_cast<uint2*>(o) = pk.u;
}

template <typename TO, int NT>
__global__ __launch_bounds__(NT) void scale_add_rmsnorm_vec_kernel(
    float* __restrict__ resid, const float* __restrict__ delta, int planes, size_t plane, float alpha,
    const float* __restrict__ w, float eps, TO* __restrict__ out, int H) {
    __shared__ float red[17];
    constexpr int ITS = 1024 / NT;
    const int r = blockIdx.x, tid = threadIdx.x, H4 = H >> 2;
    const size_t plane4 = plane >> 2;
    float4* x4 = reinterpret_cast<float4*>(resid + (size_t)r * H);
    const float4* d4 = delta ? reinterpret_cast<const float4*>(delta + (size_t)r * H) : nullptr;
    const float4* w4 = reinterpret_cast<const float4*>(w);
    auto sum_at = [&](int j) {
        float4 v = x4[j];
        v.x *= alpha; v.y *= alpha; v.z *= alpha; v.w *= alpha;
        if (d4) {
            float4 d = d4[j];
            for (int p = 1; p < planes; ++p) {
                const float4 e = d4[(size_t)p * plane4 + j];
                d.x += e.x; d.y += e.y; d.z += e.z; d.w += e.w;
            }
            v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
        }
        return v;
    };
    float4 cache[ITS];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const int j = tid + it * NT;
        if (j < H4) {
            const float4 v = sum_at(j);
            cache[it] = v;
            ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
        }
    }
    for (int j = tid + 1024; j < H4; j += NT) {
        const float4 v = sum_at(j);
        x4[j] = v;      // (kept in place for the second sweep)
        ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
    }
    ss = block_sum(ss, red);
    const float rr = 1.0f / sqrtf(ss / (float)H + eps);
    TO* o = out ? out + (size_t)r * H : nullptr;
#pragma unroll
    for (int it = 0; it < ITS; ++it) {
        const int j = tid + it * NT;
        if (j < H4) {
            const float4 v = cache[it], wv = w4[j];
            const float4 y = make_float4(v.x * rr * wv.x, v.y * rr * wv.y, v.z * rr * wv.z, v.w * rr * wv.w);
            x4[j] = y;
            if (o) pn_store4<TO>(o + 4 * j, y);
        }
    }
    for (int j = tid + 1024; j < H4; j += NT) {
        const float4 v = x4[j], wv = w4[j];
        const float4 y = make_float4(v.x * rr * wv.x, v.y * rr * wv.y, v.z * rr * wv.z, v.w * rr * wv.w);
        x4[j] = y;
        if (o) pn_store4<TO>(o + 4 * j, y);
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
    const bool vec = H % 4 == 0 && ((uintptr_t)resid % 16) == 0 && ((uintptr_t)weight % 16) == 0 &&
                     (!out || ((uintptr_t)out % 16) == 0) &&
                     (!delta || (((uintptr_t)delta % 16) == 0 && (planes == 1 || delta_plane % 4 == 0)));
    if (vec) {
        const bool wide = n <= 128 && H >= 2048;
        if (out_dtype == TFF_F32) {
            if (wide) scale_add_rmsnorm_vec_kernel<float, 1024><<<n, 1024, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps, (float*)out, H);
            else scale_add_rmsnorm_vec_kernel<float, 256><<<n, 256, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps, (float*)out, H);
        } else {
            if (wide) scale_add_rmsnorm_vec_kernel<bf16_t, 1024><<<n, 1024, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps, (bf16_t*)out, H);
            else scale_add_rmsnorm_vec_kernel<bf16_t, 256><<<n, 256, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps, (bf16_t*)out, H);
        }
        return tff_check_launch("scale_add_rmsnorm");
    }
    if (out_dtype == TFF_F32)
        scale_add_rmsnorm_kernel<float><<<n, PN_THREADS, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps,
                                                                 (float*)out, H);
    else
        scale_add_rmsnorm_kernel<bf16_t><<<n, PN_THREADS, 0, s>>>(resid, delta, planes, delta_plane, alpha, weight, eps,
                                                                  (bf16_t*)out, H);
    return tff_check_launch("scale_add_rmsnorm");
}

// form 0: gelu with erf; 1: its tanh approximation; 2: the square of relu
__device__ __forceinline__ float ffn_activation(float z, int form) {
    if (form == 2) {
        const float r = fmaxf(z, 0.f);
        return r * r;
    }
    if (form == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
}

template <typename T>
__global__ void gelu_kernel(const T* __restrict__ x, T* __restrict__ out, int64_t n, int tanh_form) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float z = to_f32(x[i]);
    out[i] = from_f32<T>(ffn_activation(z, tanh_form));
}

// bfloat16, eight elements (16 bytes) a thread
__global__ void gelu_bf16x8_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out, int64_t n8, int tanh_form) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n8) return;
    union { uint4 u; bf16_t h[8]; } a, b;
    a.u = reinterpret_cast<const uint4*>(x)[i];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float z = (float)a.h[j];
        b.h[j] = (bf16_t)ffn_activation(z, tanh_form);
    }
    reinterpret_cast<uint4*>(out)[i] = b.u;
}

TFF_API int tff_gelu(const void* x, void* out, int64_t n, int tanh_form, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(x && out, "gelu: null pointer");
    TFF_REQUIRE(n >= 0, "gelu: negative size");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == TFF_BF16 && n % 8 == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0) {
        gelu_bf16x8_kernel<<<(unsigned)((n / 8 + 255) / 256), 256, 0, s>>>((const bf16_t*)x, (bf16_t*)out, n / 8, tanh_form);
        return tff_check_launch("gelu");
    }
    if (dtype == TFF_F32)
        gelu_kernel<float><<<blocks, 256, 0, s>>>((const float*)x, (float*)out, n, tanh_form);
    else if (dtype == TFF_BF16)
        gelu_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)x, (bf16_t*)out, n, tanh_form);
    else
        return tff_fail("gelu: unknown dtype %d", dtype);
    return tff_check_launch("gelu");
}
