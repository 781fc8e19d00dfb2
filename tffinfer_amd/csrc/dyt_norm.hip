// A norm without statistics ("dynamic tanh"): y = tanh(alpha * v) * w + b, element by element, with a
// scalar alpha and vectors w, b.  No mean, no variance, no eps: a row needs no reduction, so the sum
// into the residual stream and the norm are one pass of independent elements.
//
// tff_add_dyt:  v = resid + planes of d0 + planes of d1 (each optional; the planes of a term are added in
//               their order, d0 before d1); resid <- v unless `rows` picks rows (then resid stays and only
//               those rows are normed: the model's last norm); out = tanh(alpha v) w + b in float32 or
//               bfloat16.  An element's result depends on that element alone, so it is the same bits in
//               every batch.
#include "common.h"
#include "tffinfer_kernels.h"

template <typename TO, int VEC>
__global__ __launch_bounds__(256) void add_dyt_kernel(float* __restrict__ resid, const float* __restrict__ d0, int planes0,
                                                      size_t plane0, const float* __restrict__ d1, int planes1,
                                                      size_t plane1, float alpha, const float* __restrict__ w,
                                                      const float* __restrict__ b, TO* __restrict__ out,
                                                      const int32_t* __restrict__ rows, int n, int W) {
    const int per_row = W / VEC;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)n * per_row) return;
    const int r_out = (int)(i / per_row), c = (int)(i - (size_t)r_out * per_row) * VEC;
    const int r = rows ? rows[r_out] : r_out;
    const size_t at = (size_t)r * W + c;
    float v[VEC];
    if (VEC == 4) {
        const float4 x = *reinterpret_cast<const float4*>(resid + at);
        v[0] = x.x; v[1] = x.y; v[2 % VEC] = x.z; v[3 % VEC] = x.w;
    } else {
        v[0] = resid[at];
    }
    for (int p = 0; p < planes0; ++p) {
        const float* dp = d0 + p * plane0 + at;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] += dp[e];
    }
    for (int p = 0; p < planes1; ++p) {
        const float* dp = d1 + p * plane1 + at;
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] += dp[e];
    }
    if (!rows && (planes0 > 0 || planes1 > 0)) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) resid[at + e] = v[e];
    }
    TO* o = out + (size_t)r_out * W + c;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o[e] = from_f32<TO>(fmaf(tanhf(alpha * v[e]), w[c + e], b[c + e]));
}

TFF_API int tff_add_dyt(float* resid, const float* d0, int planes0, size_t plane0, const float* d1, int planes1,
                        size_t plane1, float alpha, const float* w, const float* b, void* out, const int32_t* rows,
                        int n, int W, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(resid && w && b && out, "add_dyt: null pointer");
    TFF_REQUIRE(n >= 0 && W > 0, "add_dyt: bad sizes n=%d W=%d", n, W);
    TFF_REQUIRE((planes0 == 0 || d0) && (planes1 == 0 || d1) && planes0 >= 0 && planes1 >= 0, "add_dyt: planes without a term");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const bool vec = W % 4 == 0 && ((uintptr_t)resid % 16) == 0 && plane0 % 4 == 0 && plane1 % 4 == 0 &&
                     (!d0 || ((uintptr_t)d0 % 16) == 0) && (!d1 || ((uintptr_t)d1 % 16) == 0);
    const size_t items = (size_t)n * (vec ? W / 4 : W);
    const unsigned blocks = (unsigned)((items + 255) / 256);
#define TFF_DYT(TO, V) add_dyt_kernel<TO, V><<<blocks, 256, 0, s>>>(resid, d0, planes0, plane0, d1, planes1, plane1, alpha, w, b, (TO*)out, rows, n, W)
    if (out_dtype == TFF_F32) {
        if (vec) TFF_DYT(float, 4); else TFF_DYT(float, 1);
    } else if (out_dtype == TFF_BF16) {
        if (vec) TFF_DYT(bf16_t, 4); else TFF_DYT(bf16_t, 1);
    } else {
        return tff_fail("add_dyt: unknown dtype %d", out_dtype);
    }
#undef TFF_DYT
    return tff_check_launch("add_dyt");
}
