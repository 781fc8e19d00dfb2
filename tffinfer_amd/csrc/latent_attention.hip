// Latent attention: what stands around the paged attention kernels when keys and values are
// kept as one low-rank latent vector per token.
//
// Per token the cache holds c (kv_rank elements, RMS-normed) and one rotated key part kr
// (rot elements) that all heads share.  With the up-projections taken to the query's side,
//   score_h(i, j) = (Wuk_h^T q_h^nope)(i) . c(j) + q_h^rot(i) . kr(j)
//   out_h(i)      = Wuv_h (sum_j p_h(i, j) c(j))
// the attention itself is attention with ONE key head of size kv_rank + rot whose values are
// the first kv_rank elements of its keys, which the paged kernels of this library run as they
// are: a key page row is [c | kr | 0 ..] up to the padded head size Dp, the (transposed) value
// page holds c in its first kv_rank rows and zeros below.
//
// tff_latent_kv_store:  c = rmsnorm(x[:rank]) * w, kr = rotate(x[rank:]) into the token's slot; where the
//                       queries pass a latent vector too, its RMS norm in the same launch.
// tff_head_linear:      out[t, h, :N] = W[h] x[t, h, :K]  (W [H, N, K]), per head, with
//                       an optional sigmoid gate on the result and an optional tail of the
//                       input row that is rotated by the token's position (either pairing) and copied behind
//                       the product (the query's rotated part), zeros up to pad_to.
//                       bfloat16 on the matrix cores where rows are 16-byte aligned: a wave
//                       holds 32 tokens x 64 outputs in accumulators and reads its operands
//                       straight from memory in MFMA fragment order (eight consecutive k a
//                       lane), W as the first operand so that a lane ends up with four
//                       consecutive outputs of one token.
#include "common.h"
#include "tffinfer_kernels.h"

// Element e of the rotated part (rot elements at x, the first rot_dims of them rotated) after the rotation
// by the position's angles cs [pair][cos, sin]: pairing 0 turns (i, i + rot_dims / 2), 1 turns (2i, 2i + 1);
// the pair (u, w) becomes (u c - w s, w c + u s).
template <typename T>
__device__ __forceinline__ float latent_rotated(const T* __restrict__ x, int e, int rot_dims, int pairing,
                                                const float* __restrict__ cs) {
    const float v = to_f32(x[e]);
    if (!cs || e >= rot_dims) return v;
    int i, other;
    bool first;
    if (pairing == 0) {
        const int half = rot_dims >> 1;
        first = e < half;
        i = first ? e : e - half;
        other = first ? e + half : e - half;
    } else {
        first = !(e & 1);
        i = e >> 1;
        other = e ^ 1;
    }
    const float o = to_f32(x[other]), c = cs[2 * i], s = cs[2 * i + 1];
    return first ? fmaf(v, c, -(o * s)) : fmaf(v, c, o * s);
}

// One block a token.  xq (may be null): the query's latent vector, q_rank elements, whose RMS norm times
// q_norm_w goes to q_out.  x (may be null: a layer that reads another layer's cache): the key side.
template <typename T, typename TC>
__global__ __launch_bounds__(256) void latent_kv_store_kernel(
    const T* __restrict__ x, int x_stride, int rank, int rot, int rot_dims, int pairing,
    const float* __restrict__ norm_w, float eps, const float* __restrict__ cos_sin, int max_pos,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, TC* __restrict__ k_cache,
    TC* __restrict__ v_cache, int page_size, int Dp, const T* __restrict__ xq, int xq_stride, int q_rank,
    const float* __restrict__ q_norm_w, TC* __restrict__ q_out, int q_out_stride) {
    __shared__ float red[17];
    const int t = blockIdx.x, tid = threadIdx.x;
    if (xq) {
        const T* qr = xq + (size_t)t * xq_stride;
        float qs = 0.f;
        for (int e = tid; e < q_rank; e += blockDim.x) {
            const float v = to_f32(qr[e]);
            qs = fmaf(v, v, qs);
        }
        qs = block_sum(qs, red);
        const float rq = 1.0f / sqrtf(qs / (float)q_rank + eps);
        for (int e = tid; e < q_rank; e += blockDim.x)
            q_out[(size_t)t * q_out_stride + e] = from_f32<TC>(to_f32(qr[e]) * rq * q_norm_w[e]);
    }
    if (!x) return;
    const int slot = slots[t];
    if (slot < 0) return;      // (the whole block: a token that writes no key)
    const T* xr = x + (size_t)t * x_stride;
    float ss = 0.f;
    for (int e = tid; e < rank; e += blockDim.x) {
        const float v = to_f32(xr[e]);
        ss = fmaf(v, v, ss);
    }
    ss = block_sum(ss, red);
    const float rr = 1.0f / sqrtf(ss / (float)rank + eps);
    const int page = slot / page_size, off = slot - page * page_size;
    TC* kr = k_cache + ((size_t)page * page_size + off) * Dp;
    TC* vr = v_cache + (size_t)page * Dp * page_size + off;
    for (int e = tid; e < rank; e += blockDim.x) {
        const TC c = from_f32<TC>(to_f32(xr[e]) * rr * norm_w[e]);
        kr[e] = c;
        vr[(size_t)e * page_size] = c;
    }
    int pos = positions[t];
    pos = min(max(pos, 0), max_pos - 1);
    const float* cs = cos_sin ? cos_sin + (size_t)pos * rot_dims : nullptr;   // [pair][cos, sin]
    for (int e = tid; e < Dp - rank; e += blockDim.x)
        kr[rank + e] = from_f32<TC>(e < rot ? latent_rotated<T>(xr + rank, e, rot_dims, pairing, cs) : 0.f);
}

TFF_API int tff_latent_kv_store(const void* x, int x_stride, int T, int rank, int rot, int rot_dims, int pairing,
                                const float* norm_w, float eps, const float* cos_sin, int max_pos,
                                const int32_t* positions, const int32_t* slots, void* k_cache, void* v_cache,
                                int page_size, int num_pages, int Dp, const void* xq, int xq_stride, int q_rank,
                                const float* q_norm_w, void* q_out, int q_out_stride, int dtype, int cache_dtype,
                                tff_stream_t stream) {
    TFF_REQUIRE(x || xq, "latent_kv_store: neither a key side nor a query side");
    TFF_REQUIRE(!x || (norm_w && positions && slots && k_cache && v_cache), "latent_kv_store: null pointer");
    TFF_REQUIRE(!x || (T >= 0 && rank > 0 && rot >= 0 && Dp >= rank + rot && x_stride >= rank + rot),
                "latent_kv_store: bad sizes rank=%d rot=%d padded=%d stride=%d", rank, rot, Dp, x_stride);
    TFF_REQUIRE(!x || (rot_dims >= 0 && rot_dims <= rot && rot_dims % 2 == 0 && (rot_dims == 0 || (cos_sin && max_pos > 0)) &&
                       (pairing == 0 || pairing == 1)),
                "latent_kv_store: %d rotated dimensions of %d need an even count and a table", rot_dims, rot);
    TFF_REQUIRE(!x || (page_size > 0 && num_pages > 0), "latent_kv_store: bad cache geometry");
    TFF_REQUIRE(!xq || (q_rank > 0 && xq_stride >= q_rank && q_norm_w && q_out && q_out_stride >= q_rank),
                "latent_kv_store: the query's latent vector of %d needs a weight and a place to go", q_rank);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
#define TFF_LKS(TI, TCC)                                                                                              \
    latent_kv_store_kernel<TI, TCC><<<T, 256, 0, s>>>((const TI*)x, x_stride, rank, rot, rot_dims, pairing, norm_w, eps, \
                                                      rot_dims ? cos_sin : nullptr, max_pos, positions, slots,        \
                                                      (TCC*)k_cache, (TCC*)v_cache, page_size, Dp, (const TI*)xq,     \
                                                      xq_stride, q_rank, q_norm_w, (TCC*)q_out, q_out_stride)
    if (dtype == TFF_F32 && cache_dtype == TFF_F32)
        TFF_LKS(float, float);
    else if (dtype == TFF_BF16 && cache_dtype == TFF_BF16)
        TFF_LKS(bf16_t, bf16_t);
    else if (dtype == TFF_F32 && cache_dtype == TFF_BF16)
        TFF_LKS(float, bf16_t);
    else
        return tff_fail("latent_kv_store: rows of type %d for a cache of type %d", dtype, cache_dtype);
#undef TFF_LKS
    return tff_check_launch("latent_kv_store");
}

// ---------------------------------------------------------------- per-head products ---
// The general kernel (float32, and bfloat16 rows that are not 16-byte aligned): one block per
// (TT tokens, head, 256 output columns).  The block's input rows go to LDS as float32, KC
// elements at a time; thread n walks k along its row W[h][n][:], adding into TT accumulators,
// k ascending for every token whatever the batch.
#define HL_TT 8
#define HL_KC 128

struct HeadLinearTail {
    int tail;            // elements of the input row behind the K multiplied ones that are copied behind the product
    int rot_dims;        // of which the first rot_dims are rotated
    int pairing;         // 0: pairs (i, i + rot_dims / 2), 1: pairs (2i, 2i + 1)
    int pad_to;          // the output's head is filled with zeros up to this many elements
    int max_pos;
    const float* cos_sin;          // [position][pair][cos, sin], rot_dims / 2 pairs
    const int32_t* positions;      // per token
};

// The tail of the input heads of tokens t0 .. t0 + nt - 1 of head h, rotated and copied behind the
// N products, zeros up to pad_to; by all threads of the block.
template <typename T>
__device__ __forceinline__ void head_tail(const T* __restrict__ x, int x_row, int x_head, T* __restrict__ out,
                                          int out_row, int out_head, int t0, int nt, int h, int K, int N,
                                          const HeadLinearTail tl) {
    const int extra = tl.pad_to - N;
    for (int i = threadIdx.x; i < nt * extra; i += blockDim.x) {
        const int tt = i / extra, e = i - tt * extra;
        const T* xr = x + (size_t)(t0 + tt) * x_row + (size_t)h * x_head + K;
        float v = 0.f;
        if (e < tl.tail) {
            if (e < tl.rot_dims) {
                const int pos = min(max(tl.positions[t0 + tt], 0), tl.max_pos - 1);
                v = latent_rotated<T>(xr, e, tl.rot_dims, tl.pairing, tl.cos_sin + (size_t)pos * tl.rot_dims);
            } else {
                v = to_f32(xr[e]);
            }
        }
        out[(size_t)(t0 + tt) * out_row + (size_t)h * out_head + N + e] = from_f32<T>(v);
    }
}

template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(
    const T* __restrict__ x, int x_row, int x_head, const T* __restrict__ Wt, T* __restrict__ out, int out_row,
    int out_head, int Tn, int K, int N, const T* __restrict__ gate, int gate_row, HeadLinearTail tl) {
    __shared__ float xs[HL_TT][HL_KC];
    const int t0 = blockIdx.x * HL_TT, h = blockIdx.y, tid = threadIdx.x;
    const int n = blockIdx.z * 256 + tid;
    const int nt = min(HL_TT, Tn - t0);
    const T* W = Wt + ((size_t)h * N + min(n, N - 1)) * K;      // the thread's row
    float acc[HL_TT];
#pragma unroll
    for (int i = 0; i < HL_TT; ++i) acc[i] = 0.f;
    for (int k0 = 0; k0 < K; k0 += HL_KC) {
        const int kc = min(HL_KC, K - k0);
        __syncthreads();
        for (int i = tid; i < HL_TT * HL_KC; i += 256) {
            const int tt = i / HL_KC, k = i - tt * HL_KC;
            xs[tt][k] = (tt < nt && k < kc) ? to_f32(x[(size_t)(t0 + tt) * x_row + (size_t)h * x_head + k0 + k]) : 0.f;
        }
        __syncthreads();
        if (n < N) {
            for (int k = 0; k < kc; ++k) {
                const float w = to_f32(W[k0 + k]);
#pragma unroll
                for (int i = 0; i < HL_TT; ++i) acc[i] = fmaf(xs[i][k], w, acc[i]);
            }
        }
    }
    if (n < N) {
#pragma unroll
        for (int i = 0; i < HL_TT; ++i) {
            if (i >= nt) break;
            float v = acc[i];
            if (gate) {
                const float gz = to_f32(gate[(size_t)(t0 + i) * gate_row + (size_t)h * N + n]);
                v *= 1.0f / (1.0f + expf(-gz));
            }
            out[(size_t)(t0 + i) * out_row + (size_t)h * out_head + n] = from_f32<T>(v);
        }
    }
    if (blockIdx.z == 0 && tl.pad_to > N) head_tail<T>(x, x_row, x_head, out, out_row, out_head, t0, nt, h, K, N, tl);
}

// bfloat16 on the matrix cores.  Block: 128 tokens x 64 outputs of one head, four waves of 32
// tokens each.  C[n][t] += W[n][k] x[t][k]: W's rows are the first operand's rows, so lane
// (t = lane & 15, kg = lane >> 4) holds outputs n = kg * 4 .. + 3 of token t for each of the
// 4 x 2 tiles.  k ascends in steps of 32 for every token whatever the batch.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 hl_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float hl_floatx4;

__device__ __forceinline__ hl_bf16x8 hl_load8(const bf16_t* p, bool ok) {
    union { uint4 u; hl_bf16x8 v; } x;
    x.u = ok ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
    return x.v;
}

__global__ __launch_bounds__(256) void head_linear_mfma_kernel(
    const bf16_t* __restrict__ x, int x_row, int x_head, const bf16_t* __restrict__ W, bf16_t* __restrict__ out,
    int out_row, int out_head, int Tn, int K, int N, const bf16_t* __restrict__ gate, int gate_row,
    HeadLinearTail tl) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, r = lane & 15, kg = lane >> 4;
    const int h = blockIdx.y, n0 = blockIdx.z * 64;
    const int tb = blockIdx.x * 128, t0 = tb + wv * 32;
    hl_floatx4 acc[4][2];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 2; ++i) acc[j][i] = hl_floatx4{0.f, 0.f, 0.f, 0.f};
    const bf16_t* xp[2];
    bool xok[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int t = t0 + i * 16 + r;
        xok[i] = t < Tn;
        xp[i] = x + (size_t)min(t, Tn - 1) * x_row + (size_t)h * x_head + kg * 8;
    }
    const bf16_t* wp[4];
    bool wok[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = n0 + j * 16 + r;
        wok[j] = n < N;
        wp[j] = W + ((size_t)h * N + min(n, N - 1)) * K + kg * 8;
    }
    if (t0 < Tn) {      // (a wave's condition: the MFMAs below run for whole waves)
        for (int k0 = 0; k0 < K; k0 += 32) {
            const bool kok = k0 + kg * 8 < K;      // K is a multiple of 8: a lane's eight elements exist together
            hl_bf16x8 a[4], b[2];
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = hl_load8(wp[j] + k0, wok[j] && kok);
#pragma unroll
            for (int i = 0; i < 2; ++i) b[i] = hl_load8(xp[i] + k0, xok[i] && kok);
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 2; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], b[i], acc[j][i], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int t = t0 + i * 16 + r;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float v4[4] = {acc[j][i][0], acc[j][i][1], acc[j][i][2], acc[j][i][3]};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int n = n0 + j * 16 + kg * 4 + e;
                    if (t < Tn && n < N) {
                        float v = v4[e];
                        if (gate) {
                            const float gz = (float)gate[(size_t)t * gate_row + (size_t)h * N + n];
                            v *= 1.0f / (1.0f + expf(-gz));
                        }
                        out[(size_t)t * out_row + (size_t)h * out_head + n] = (bf16_t)v;
                    }
                }
            }
        }
    }
    if (blockIdx.z == 0 && tl.pad_to > N)
        head_tail<bf16_t>(x, x_row, x_head, out, out_row, out_head, tb, min(128, Tn - tb), h, K, N, tl);
}

TFF_API int tff_head_linear(const void* x, int x_row, int x_head, const void* Wt, void* out, int out_row, int out_head,
                            int T, int H, int K, int N, const void* gate, int gate_row, int tail, int rot_dims,
                            int pairing, int pad_to, const float* cos_sin, int max_pos, const int32_t* positions, int dtype,
                            tff_stream_t stream) {
    TFF_REQUIRE(x && Wt && out, "head_linear: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && K > 0 && N > 0 && H <= 65535, "head_linear: bad sizes T=%d H=%d K=%d N=%d", T, H, K, N);
    TFF_REQUIRE(x_head >= K + tail && x_row >= (H - 1) * x_head + K + tail,
                "head_linear: input rows of %d with heads %d apart do not hold %d heads of %d + %d", x_row, x_head, H, K, tail);
    const int width = pad_to > N ? pad_to : N;
    TFF_REQUIRE(tail >= 0 && width >= N + tail && out_head >= width && out_row >= (H - 1) * out_head + width,
                "head_linear: output rows of %d with heads %d apart do not hold %d heads of %d", out_row, out_head, H, width);
    TFF_REQUIRE(rot_dims >= 0 && rot_dims <= tail && rot_dims % 2 == 0 && (rot_dims == 0 || (cos_sin && positions && max_pos > 0)) &&
                (pairing == 0 || pairing == 1),
                "head_linear: %d rotated dimensions of a tail of %d need an even count, a table and positions", rot_dims, tail);
    TFF_REQUIRE(!gate || gate_row >= H * N, "head_linear: gate rows of %d hold fewer than %d", gate_row, H * N);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const HeadLinearTail tl{tail, rot_dims, pairing, pad_to, max_pos, cos_sin, positions};
    const dim3 grid((T + HL_TT - 1) / HL_TT, H, (N + 255) / 256);
    if (dtype == TFF_F32)
        head_linear_kernel<float><<<grid, 256, 0, s>>>((const float*)x, x_row, x_head, (const float*)Wt, (float*)out, out_row,
                                                       out_head, T, K, N, (const float*)gate, gate_row, tl);
    else if (dtype == TFF_BF16) {
        const bool aligned = K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && ((uintptr_t)x % 16) == 0 &&
                             ((uintptr_t)Wt % 16) == 0;
        if (aligned)
            head_linear_mfma_kernel<<<dim3((T + 127) / 128, H, (N + 63) / 64), 256, 0, s>>>(
                (const bf16_t*)x, x_row, x_head, (const bf16_t*)Wt, (bf16_t*)out, out_row, out_head, T, K, N,
                (const bf16_t*)gate, gate_row, tl);
        else
            head_linear_kernel<bf16_t><<<grid, 256, 0, s>>>((const bf16_t*)x, x_row, x_head, (const bf16_t*)Wt, (bf16_t*)out,
                                                            out_row, out_head, T, K, N, (const bf16_t*)gate, gate_row, tl);
    }
    else
        return tff_fail("head_linear: unknown dtype %d", dtype);
    return tff_check_launch("head_linear");
}
