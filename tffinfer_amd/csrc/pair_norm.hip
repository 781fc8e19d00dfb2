// The norms of a layer whose mixer and feed-forward read the same rows, and the cap on the logits.
//
// tff_add_rmsnorm_pair: v = resid + (the planes of d0, in order) + (the planes of d1, in order) + bias, per row;
//   resid <- v (unless `rows` picks rows: then resid stays as it is and only those rows are normed);
//   out1 = v * rsqrt(mean(v^2) + eps) * w1, and out2 the same with w2 when a second weight is given.
//   Every term is optional.  Sums and norms in float32; one block a row, the row kept in LDS.
// tff_softcap: z <- cap * tanh(z / cap), in place, float32.
#include "common.h"
#include "tffinfer_kernels.h"

#define PN_MAX_W 15360

// NT threads a block: 256 where the rows fill the GPU, 1024 for the few rows of a decode step (four elements a
// thread instead of sixteen, so that a row's loads are in flight together).  The sum of squares is formed by the
// first 256 threads from LDS, element e by thread e mod 256 in the order of e, whatever NT is: a row's norm does
// not depend on how many rows the step has.
template <typename TO, int NT>
__global__ __launch_bounds__(NT) void add_rmsnorm_pair_kernel(
    float* __restrict__ resid, const float* __restrict__ d0, int planes0, size_t plane0, const float* __restrict__ d1,
    int planes1, size_t plane1, const float* __restrict__ bias, const float* __restrict__ w1, const float* __restrict__ w2,
    float eps, TO* __restrict__ out1, TO* __restrict__ out2, const int32_t* __restrict__ rows, int W) {
    extern __shared__ float vrow[];
    __shared__ float red[17];
    const int i = blockIdx.x;
    const size_t row = rows ? (size_t)rows[i] : (size_t)i;
    float* x = resid + row * W;
    for (int e = threadIdx.x; e < W; e += NT) {
        float v = x[e];
#pragma unroll 4
        for (int p = 0; p < planes0; ++p) v += d0[p * plane0 + row * W + e];
#pragma unroll 4
        for (int p = 0; p < planes1; ++p) v += d1[p * plane1 + row * W + e];
        if (bias) v += bias[e];
        if (!rows) x[e] = v;
        vrow[e] = v;
    }
    __syncthreads();
    float ss = 0.f;
    if (threadIdx.x < 256)
        for (int e = threadIdx.x; e < W; e += 256) ss = fmaf(vrow[e], vrow[e], ss);
    ss = block_sum(ss, red);
    const float rr = 1.0f / sqrtf(ss / (float)W + eps);
    for (int e = threadIdx.x; e < W; e += NT) {
        const float v = vrow[e] * rr;
        out1[(size_t)i * W + e] = from_f32<TO>(v * w1[e]);
        if (w2) out2[(size_t)i * W + e] = from_f32<TO>(v * w2[e]);
    }
}

TFF_API int tff_add_rmsnorm_pair(float* resid, const float* d0, int planes0, size_t plane0, const float* d1, int planes1,
                                 size_t plane1, const float* bias, const float* w1, const float* w2, float eps, void* out1,
                                 void* out2, const int32_t* rows, int n, int W, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(resid && w1 && out1 && (!w2 || out2), "add_rmsnorm_pair: null pointer");
    TFF_REQUIRE(n >= 0 && W > 0 && W <= PN_MAX_W, "add_rmsnorm_pair: rows of %d (up to %d)", W, PN_MAX_W);
    TFF_REQUIRE((d0 ? planes0 >= 1 : planes0 == 0) && (d1 ? planes1 >= 1 : planes1 == 0), "add_rmsnorm_pair: planes without a term");
    if (n == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t lds = (size_t)W * sizeof(float);
#define PN_LAUNCH(TO, NT)                                                                                              \
    add_rmsnorm_pair_kernel<TO, NT><<<n, NT, lds, s>>>(resid, d0, planes0, plane0, d1, planes1, plane1, bias, w1, w2, eps, \
                                                      (TO*)out1, (TO*)out2, rows, W)
    const bool few = n <= 128 && W > 1024;
    if (out_dtype == TFF_F32) {
        if (few) PN_LAUNCH(float, 1024); else PN_LAUNCH(float, 256);
    } else if (out_dtype == TFF_BF16) {
        if (few) PN_LAUNCH(bf16_t, 1024); else PN_LAUNCH(bf16_t, 256);
    } else
        return tff_fail("add_rmsnorm_pair: unknown dtype %d", out_dtype);
#undef PN_LAUNCH
    return tff_check_launch("add_rmsnorm_pair");
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ z, float cap, float inv, size_t count) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < count) z[i] = cap * tanhf(z[i] * inv);
}

TFF_API int tff_softcap(float* z, size_t count, float cap, tff_stream_t stream) {
    TFF_REQUIRE(z, "softcap: null pointer");
    TFF_REQUIRE(cap > 0.f, "softcap: the cap must be positive");
    if (count == 0) return 0;
    softcap_kernel<<<(unsigned)((count + 255) / 256), 256, 0, (hipStream_t)stream>>>(z, cap, 1.0f / cap, count);
    return tff_check_launch("softcap");
}
