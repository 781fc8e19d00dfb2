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
//   sum is fixed by the head size and the kernel's form alone, so a token's result does not depend on
//   how the tokens were cut into steps beyond rounding (`long_portions` picks the form for prompts, whose
//   sums run in another order than those of the form for single tokens).  The block of head 0 also
//   leaves the portion's last row of x in the state.
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
    const int c = blockIdx.y * 256 + threadIdx.x;      // (a block a token and 256 columns: few tokens still fill the GPU)
    if (c < W) {
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
    const dim3 grid(T, (W + 255) / 256);
    if (out_dtype == TFF_F32)
        token_shift_mix_kernel<float><<<grid, 256, 0, s>>>(x, state, state_row, prev_off, mu, M, token_req, cu_tokens,
                                                         state_slots, (float*)out, T, W);
    else if (out_dtype == TFF_BF16)
        token_shift_mix_kernel<bf16_t><<<grid, 256, 0, s>>>(x, state, state_row, prev_off, mu, M, token_req, cu_tokens,
                                                          state_slots, (bf16_t*)out, T, W);
    else
        return tff_fail("token_shift_mix: unknown dtype %d", out_dtype);
    return tff_check_launch("token_shift_mix");
}

#define WKV_MAX_D 128     // (a thread keeps a slice of a column of S in registers)
#define WKV_MAX_SLICES 4
#define WKV_CHUNK_ELEMS 1024   // tokens of a chunk x padded head size, at most
#define WKV_EPT 4              // elements of a chunk's array a thread fetches, at most

// KPT key channels a thread; ceil(D / KPT) <= 4 slices of the key channels; thread = slice * D + value channel.
// The tokens of a portion pass in chunks of up to 16: a chunk's r, k, w, v are fetched into registers while the
// chunk before it is worked through from LDS, so that no token waits for memory; within a chunk a token costs
// its multiply-adds, its slice of r, k, w in 16-byte LDS reads and one barrier (the slices' partial sums meet
// in LDS, in a buffer of the token's parity).  In LDS a token's channels lie Dp = slices * KPT apart, the
// channels past D zero, so that a slice needs no bounds.
template <int KPT>
__global__ __launch_bounds__(512) void wkv_recurrence_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ z, size_t row, const float* __restrict__ w0, const float* __restrict__ u,
    float* __restrict__ state, size_t state_row, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ state_slots, float* __restrict__ o, int H, int D, const float* __restrict__ x, int W,
    size_t prev_off) {
    __shared__ __attribute__((aligned(16))) float buf[2][3][WKV_CHUNK_ELEMS];       // r, k, w of a chunk, [token][channel]
    __shared__ float bv[2][WKV_CHUNK_ELEMS];                                       // v of a chunk
    __shared__ float so[WKV_CHUNK_ELEMS];
    __shared__ float part[2][WKV_MAX_SLICES][WKV_MAX_D];
    const int h = blockIdx.x, req = blockIdx.y, tid = threadIdx.x, nt = blockDim.x;
    const int t0 = cu_tokens[req], t1 = cu_tokens[req + 1];
    if (t1 <= t0) return;
    const int slices = nt / D;
    const int Dp = slices * KPT;
    const int vi = tid % D, ks = tid / D;
    const int C = min(min(16, WKV_EPT * slices), WKV_CHUNK_ELEMS / Dp);      // tokens a chunk
    float* srow = state + (size_t)state_slots[req] * state_row;
    float* S = srow + (size_t)h * D * D;
    const size_t col = (size_t)h * D;
    float s[KPT], uu[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int kk = ks * KPT + i;
        s[i] = kk < D ? S[(size_t)kk * D + vi] : 0.f;
        uu[i] = kk < D ? u[col + kk] : 0.f;
    }
    for (int e = tid; e < 2 * 3 * WKV_CHUNK_ELEMS; e += nt) (&buf[0][0][0])[e] = 0.f;      // (the channels past D stay zero)
    float fr[WKV_EPT], fk[WKV_EPT], fz[WKV_EPT], fv[WKV_EPT];
    // a chunk's elements e = token * D + channel are dealt to the threads in strides of the block
    auto fetch = [&](int base) {
        const int n = min(C, t1 - base) * D;
#pragma unroll
        for (int i = 0; i < WKV_EPT; ++i) {
            const int e = tid + i * nt;
            if (e < n) {
                const size_t a = (size_t)(base + e / D) * row + col + e % D;
                fr[i] = r[a];
                fk[i] = k[a];
                fz[i] = z[a] + w0[col + e % D];
                fv[i] = v[a];
            }
        }
    };
    auto stage = [&](int base, int b) {
        const int n = min(C, t1 - base) * D;
#pragma unroll
        for (int i = 0; i < WKV_EPT; ++i) {
            const int e = tid + i * nt;
            if (e < n) {
                const int at = (e / D) * Dp + e % D;
                buf[b][0][at] = fr[i];
                buf[b][1][at] = fk[i];
                buf[b][2][at] = expf(-expf(fz[i]));
                bv[b][e] = fv[i];
            }
        }
    };
    fetch(t0);
    __syncthreads();
    stage(t0, 0);
    int b = 0;
    for (int base = t0; base < t1; base += C, b ^= 1) {
        const int n = min(C, t1 - base);
        __syncthreads();
        if (base + C < t1) fetch(base + C);
        for (int c = 0; c < n; ++c) {
            const float4* cr = reinterpret_cast<const float4*>(buf[b][0] + c * Dp + ks * KPT);
            const float4* ck = reinterpret_cast<const float4*>(buf[b][1] + c * Dp + ks * KPT);
            const float4* cw = reinterpret_cast<const float4*>(buf[b][2] + c * Dp + ks * KPT);
            const float vt = bv[b][c * D + vi];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < KPT; i += 4) {
                const float4 r4 = cr[i >> 2], k4 = ck[i >> 2], w4 = cw[i >> 2];
                const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk4[4] = {k4.x, k4.y, k4.z, k4.w},
                            ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float kv = kk4[j] * vt;
                    acc = fmaf(rr[j], fmaf(uu[i + j], kv, s[i + j]), acc);
                    s[i + j] = fmaf(ww[j], s[i + j], kv);
                }
            }
            part[c & 1][ks][vi] = acc;
            __syncthreads();
            if (ks == 0) {
                float sum = part[c & 1][0][vi];
                for (int p = 1; p < slices; ++p) sum += part[c & 1][p][vi];
                so[c * D + vi] = sum;
            }
        }
        __syncthreads();
        for (int e = tid; e < n * D; e += nt) o[(size_t)(base + e / D) * H * D + col + e % D] = so[e];
        if (base + C < t1) stage(base + C, b ^ 1);
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        const int kk = ks * KPT + i;
        if (kk < D) S[(size_t)kk * D + vi] = s[i];
    }
    if (h == 0 && x) {
        const float* last = x + (size_t)(t1 - 1) * W;
        for (int c = tid; c < W; c += nt) srow[prev_off + c] = last[c];
    }
}

// The same for head sizes that are multiples of 16 (D = 4 * KPT): a wave takes sixteen value channels, its four
// rows of sixteen lanes a quarter of the key channels each, and the quarters' partial sums meet through lane
// swaps: no barrier and no LDS between the tokens of a chunk, the waves run on their own.
template <int KPT>
__global__ __launch_bounds__(512) void wkv_recurrence_wave_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ z, size_t row, const float* __restrict__ w0, const float* __restrict__ u,
    float* __restrict__ state, size_t state_row, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ state_slots, float* __restrict__ o, int H, const float* __restrict__ x, int W,
    size_t prev_off) {
    constexpr int D = 4 * KPT;
    constexpr int C = (WKV_CHUNK_ELEMS / D) < 16 ? (WKV_CHUNK_ELEMS / D) : 16;      // tokens a chunk
    constexpr int NT = 4 * D;                                                      // threads: D / 16 waves
    constexpr int EPT = (C * D + NT - 1) / NT;
    __shared__ __attribute__((aligned(16))) float buf[2][3][C * D];       // r, k, w of a chunk, [token][channel]
    __shared__ float bv[2][C * D];
    const int h = blockIdx.x, req = blockIdx.y, tid = threadIdx.x;
    const int t0 = cu_tokens[req], t1 = cu_tokens[req + 1];
    if (t1 <= t0) return;
    const int lane = tid & 63;
    const int ks = lane >> 4, vi = (tid >> 6) * 16 + (lane & 15);
    float* srow = state + (size_t)state_slots[req] * state_row;
    float* S = srow + (size_t)h * D * D;
    const size_t col = (size_t)h * D;
    float s[KPT], uu[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        s[i] = S[(size_t)(ks * KPT + i) * D + vi];
        uu[i] = u[col + ks * KPT + i];
    }
    float fr[EPT], fk[EPT], fz[EPT], fv[EPT];
    auto fetch = [&](int base) {
        const int n = min(C, t1 - base) * D;
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * NT;
            if (e < n) {
                const size_t a = (size_t)(base + e / D) * row + col + e % D;
                fr[i] = r[a];
                fk[i] = k[a];
                fz[i] = z[a] + w0[col + e % D];
                fv[i] = v[a];
            }
        }
    };
    auto stage = [&](int base, int b) {
        const int n = min(C, t1 - base) * D;
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * NT;
            if (e < n) {
                buf[b][0][e] = fr[i];
                buf[b][1][e] = fk[i];
                buf[b][2][e] = expf(-expf(fz[i]));
                bv[b][e] = fv[i];
            }
        }
    };
    fetch(t0);
    stage(t0, 0);
    int b = 0;
    for (int base = t0; base < t1; base += C, b ^= 1) {
        const int n = min(C, t1 - base);
        __syncthreads();
        if (base + C < t1) fetch(base + C);
        for (int c = 0; c < n; ++c) {
            const float4* cr = reinterpret_cast<const float4*>(buf[b][0] + c * D + ks * KPT);
            const float4* ck = reinterpret_cast<const float4*>(buf[b][1] + c * D + ks * KPT);
            const float4* cw = reinterpret_cast<const float4*>(buf[b][2] + c * D + ks * KPT);
            const float vt = bv[b][c * D + vi];
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < KPT; i += 4) {
                const float4 r4 = cr[i >> 2], k4 = ck[i >> 2], w4 = cw[i >> 2];
                const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk4[4] = {k4.x, k4.y, k4.z, k4.w},
                            ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float kv = kk4[j] * vt;
                    acc = fmaf(rr[j], fmaf(uu[i + j], kv, s[i + j]), acc);
                    s[i + j] = fmaf(ww[j], s[i + j], kv);
                }
            }
            acc = rows_sum(acc);        // (quarter 0 + quarter 1) + (quarter 2 + quarter 3), in every lane
            if (ks == 0) o[(size_t)(base + c) * H * D + col + vi] = acc;
        }
        // (the other buffer was last read before this pass's barrier)
        if (base + C < t1) stage(base + C, b ^ 1);
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) S[(size_t)(ks * KPT + i) * D + vi] = s[i];
    if (h == 0 && x) {
        const float* last = x + (size_t)(t1 - 1) * W;
        for (int c = tid; c < W; c += NT) srow[prev_off + c] = last[c];
    }
}

// For long portions (prompts) of heads of 64 or 128 channels (D = 16 * KPT): a token's cost is what bounds a
// prompt, since its tokens go one after the other.  Here a row of sixteen lanes shares a value channel, each
// lane KPT key channels, so a token is KPT steps of four instructions and a sum over the row; a block of four
// waves takes sixteen value channels of a head, D / 16 blocks a head.
template <int KPT>
__global__ __launch_bounds__(256) void wkv_recurrence_rows_kernel(
    const float* __restrict__ r, const float* __restrict__ k, const float* __restrict__ v,
    const float* __restrict__ z, size_t row, const float* __restrict__ w0, const float* __restrict__ u,
    float* __restrict__ state, size_t state_row, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ state_slots, float* __restrict__ o, int H, const float* __restrict__ x, int W,
    size_t prev_off) {
    constexpr int D = 16 * KPT;
    constexpr int C = WKV_CHUNK_ELEMS / D;         // tokens a chunk: 16 or 8
    constexpr int NT = 256;
    constexpr int EPT = C * D / NT;                // 4
    constexpr int Q = KPT / 4;
    __shared__ __attribute__((aligned(16))) float buf[2][3][C * D];       // r, k, w of a chunk, [token][channel]
    __shared__ float bv[2][C * 16];                                        // v of the block's sixteen channels
    const int h = blockIdx.x, req = blockIdx.y, tid = threadIdx.x;
    const int t0 = cu_tokens[req], t1 = cu_tokens[req + 1];
    if (t1 <= t0) return;
    const int lane = tid & 63;
    const int ks = lane & 15, vl = (tid >> 6) * 4 + (lane >> 4), vi = blockIdx.z * 16 + vl;
    float* srow = state + (size_t)state_slots[req] * state_row;
    float* S = srow + (size_t)h * D * D;
    const size_t col = (size_t)h * D;
    float s[KPT], uu[KPT];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
        s[i] = S[(size_t)(ks * KPT + i) * D + vi];
        uu[i] = u[col + ks * KPT + i];
    }
    float fr[EPT], fk[EPT], fz[EPT], fv = 0.f;
    auto fetch = [&](int base) {
        const int n = min(C, t1 - base);
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * NT;
            if (e < n * D) {
                const size_t a = (size_t)(base + e / D) * row + col + e % D;
                fr[i] = r[a];
                fk[i] = k[a];
                fz[i] = z[a] + w0[col + e % D];
            }
        }
        if (tid < n * 16) fv = v[(size_t)(base + tid / 16) * row + col + blockIdx.z * 16 + tid % 16];
    };
    auto stage = [&](int base, int b) {
        const int n = min(C, t1 - base);
#pragma unroll
        for (int i = 0; i < EPT; ++i) {
            const int e = tid + i * NT;
            if (e < n * D) {
                buf[b][0][e] = fr[i];
                buf[b][1][e] = fk[i];
                buf[b][2][e] = expf(-expf(fz[i]));
            }
        }
        if (tid < n * 16) bv[b][tid] = fv;
    };
    fetch(t0);
    stage(t0, 0);
    int b = 0;
    for (int base = t0; base < t1; base += C, b ^= 1) {
        const int n = min(C, t1 - base);
        __syncthreads();
        if (base + C < t1) fetch(base + C);
        // (unrolled by four: only s runs from token to token, one multiply-add an element; the sums over the rows,
        // the stores and the LDS reads of neighbouring tokens overlap)
        float* orow = o + (size_t)base * H * D + col + vi;
#pragma unroll 4
        for (int c = 0; c < n; ++c) {
            const float4* cr = reinterpret_cast<const float4*>(buf[b][0] + c * D + ks * KPT);
            const float4* ck = reinterpret_cast<const float4*>(buf[b][1] + c * D + ks * KPT);
            const float4* cw = reinterpret_cast<const float4*>(buf[b][2] + c * D + ks * KPT);
            const float vt = bv[b][c * 16 + vl];
            float acc = 0.f;
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                const float4 r4 = cr[q], k4 = ck[q], w4 = cw[q];
                const float rr[4] = {r4.x, r4.y, r4.z, r4.w}, kk4[4] = {k4.x, k4.y, k4.z, k4.w},
                            ww[4] = {w4.x, w4.y, w4.z, w4.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const float kv = kk4[j] * vt;
                    acc = fmaf(rr[j], fmaf(uu[4 * q + j], kv, s[4 * q + j]), acc);
                    s[4 * q + j] = fmaf(ww[j], s[4 * q + j], kv);
                }
            }
            acc = row16_sum(acc);
            if (ks == 0) orow[(size_t)c * H * D] = acc;
        }
        // (the other buffer was last read before this pass's barrier)
        if (base + C < t1) stage(base + C, b ^ 1);
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) S[(size_t)(ks * KPT + i) * D + vi] = s[i];
    if (h == 0 && blockIdx.z == 0 && x) {
        const float* last = x + (size_t)(t1 - 1) * W;
        for (int c = tid; c < W; c += NT) srow[prev_off + c] = last[c];
    }
}

TFF_API int tff_wkv_recurrence(const float* r, const float* k, const float* v, const float* z, size_t row, const float* w0,
                               const float* u, float* state, size_t state_row, const int32_t* cu_tokens,
                               const int32_t* state_slots, float* o, int R, int H, int D, const float* x, int W,
                               size_t prev_off, int long_portions, tff_stream_t stream) {
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
#define WKV_WAVES(KPT)                                                                                             \
    wkv_recurrence_wave_kernel<KPT><<<grid, 16 * KPT, 0, s>>>(r, k, v, z, row, w0, u, state, state_row, cu_tokens, \
                                                              state_slots, o, H, x, W, prev_off)
    if (long_portions && (D == 64 || D == 128)) {
        const dim3 grid3(H, R, D / 16);
        if (D == 64)
            wkv_recurrence_rows_kernel<4><<<grid3, 256, 0, s>>>(r, k, v, z, row, w0, u, state, state_row, cu_tokens,
                                                                state_slots, o, H, x, W, prev_off);
        else
            wkv_recurrence_rows_kernel<8><<<grid3, 256, 0, s>>>(r, k, v, z, row, w0, u, state, state_row, cu_tokens,
                                                                state_slots, o, H, x, W, prev_off);
    } else if (D % 16 == 0) {
        switch (D / 4) {
            case 4: WKV_WAVES(4); break;
            case 8: WKV_WAVES(8); break;
            case 12: WKV_WAVES(12); break;
            case 16: WKV_WAVES(16); break;
            case 20: WKV_WAVES(20); break;
            case 24: WKV_WAVES(24); break;
            case 28: WKV_WAVES(28); break;
            default: WKV_WAVES(32); break;
        }
    } else if (D <= 64) WKV_LAUNCH(16);
    else WKV_LAUNCH(32);
#undef WKV_WAVES
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
