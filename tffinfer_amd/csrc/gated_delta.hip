// The gated delta rule: a linear recurrence whose state, a matrix S [key channel, value channel]
// per request and head, is decayed, corrected towards the token's value along the token's key,
// and read with the token's query:
//
//   S <- g_t S;   u_t = beta_t (v_t - S^T k_t);   S <- S + k_t u_t^T;   o_t = S^T q_t
//
// with g_t = exp(-exp(A) softplus(a_t + dt)) and beta_t = sigmoid(b_t) per head, k_t a unit vector,
// q_t a unit vector times dim^(-1/2).  q, k, v come from a projection through a short causal
// convolution over time per channel and silu; the convolution's last taps - 1 inputs are part of
// the request's state, behind the heads' matrices.  Everything here is float32.
//
// A request's state row: [heads][value channel][key channel] (S transposed: the key channels of one
// value channel lie side by side, as the lanes that share the channel read them), then
// [taps - 1][channels] of the convolution's inputs, oldest first; channels are q (kv_heads x dim),
// k (kv_heads x dim), v (heads x vdim), in the projection's column order.
//
// tff_gdelta_prep:        per token: convolution + silu of q, k, v, unit vectors, beta and the decay.
// tff_gdelta_recurrence:  the recurrence over each request's tokens of the step; also leaves the
//                         convolution's last inputs in the state.
// tff_head_norm_silu_gate: out = o / sqrt(mean over the head of o^2 + eps) * w[channel] * silu(gate).
// tff_sigmoid_gate_heads: out = o * sigmoid(gate) * scale, heads of o a stride apart.
#include "common.h"
#include "tffinfer_kernels.h"

#define GD_MAX_TAPS 8
#define GD_FEW 4        // tokens a request up to which a step counts as decoding

__device__ __forceinline__ float gd_silu(float z) { return z / (1.0f + expf(-z)); }

// One wave per (token, unit); units: kv_heads q heads, kv_heads k heads, heads v heads, one for beta and decay.
__global__ __launch_bounds__(64) void gdelta_prep_kernel(
    const float* __restrict__ proj, size_t ldp, const float* __restrict__ wconv, int taps,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, const float* __restrict__ state,
    size_t state_row, size_t tail_off, const int32_t* __restrict__ token_req, const int32_t* __restrict__ cu_tokens,
    const int32_t* __restrict__ state_slots, float* __restrict__ pre, int H, int G, int D, int E) {
    const int t = blockIdx.x, u = blockIdx.y, lane = threadIdx.x;
    const int C = 2 * G * D + H * E;
    const size_t ldq = (size_t)C + 2 * H;
    const float* row = proj + (size_t)t * ldp;
    float* out = pre + (size_t)t * ldq;
    if (u == 2 * G + H) {
        for (int h = lane; h < H; h += 64) {
            const float b = row[C + h], a = row[C + H + h] + dt_bias[h];
            const float sp = a > 20.f ? a : log1pf(expf(a));
            out[C + h] = 1.0f / (1.0f + expf(-b));
            out[C + H + h] = expf(-expf(a_log[h]) * sp);
        }
        return;
    }
    const int r = token_req[t];
    const int i = t - cu_tokens[r];               // the token's place in its request's portion
    const float* tail = state + (size_t)state_slots[r] * state_row + tail_off;
    int c0, n;
    if (u < 2 * G) { c0 = u * D; n = D; } else { c0 = 2 * G * D + (u - 2 * G) * E; n = E; }
    float ss = 0.f;
    for (int e = lane; e < n; e += 64) {
        const int c = c0 + e;
        float acc = 0.f;
        for (int k = 0; k < taps; ++k) {
            const int s = i - (taps - 1) + k;     // the input's place in the portion; before it: the state's
            const float x = s >= 0 ? proj[(size_t)(t - (taps - 1) + k) * ldp + c] : tail[(size_t)(i + k) * C + c];
            acc = fmaf(wconv[(size_t)c * taps + k], x, acc);
        }
        const float y = gd_silu(acc);
        out[c] = y;
        ss = fmaf(y, y, ss);
    }
    if (u < 2 * G) {
        ss = wave_sum(ss);
        const float f = (1.0f / sqrtf(ss + 1e-6f)) * (u < G ? 1.0f / sqrtf((float)D) : 1.0f);
        __syncthreads();
        for (int e = lane; e < n; e += 64) out[c0 + e] *= f;      // (each lane rescales what it wrote)
    }
}

TFF_API int tff_gdelta_prep(const float* proj, size_t ldp, const float* wconv, int taps, const float* a_log,
                            const float* dt_bias, const float* state, size_t state_row, size_t tail_off,
                            const int32_t* token_req, const int32_t* cu_tokens, const int32_t* state_slots, float* pre,
                            int T, int H, int G, int D, int E, tff_stream_t stream) {
    TFF_REQUIRE(proj && wconv && a_log && dt_bias && state && token_req && cu_tokens && state_slots && pre,
                "gdelta_prep: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && E > 0 && taps >= 1 && taps <= GD_MAX_TAPS,
                "gdelta_prep: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d taps=%d (taps up to %d)", H, G, D, E, taps,
                GD_MAX_TAPS);
    const size_t C = 2 * (size_t)G * D + (size_t)H * E;
    TFF_REQUIRE(ldp >= C + 2 * (size_t)H && tail_off + (size_t)(taps - 1) * C <= state_row,
                "gdelta_prep: rows of %zu or state rows of %zu are too short", ldp, state_row);
    TFF_REQUIRE(2 * G + H + 1 <= 65535, "gdelta_prep: too many heads");
    if (T == 0) return 0;
    gdelta_prep_kernel<<<dim3(T, 2 * G + H + 1), 64, 0, (hipStream_t)stream>>>(
        proj, ldp, wconv, taps, a_log, dt_bias, state, state_row, tail_off, token_req, cu_tokens, state_slots, pre, H, G, D, E);
    return tff_check_launch("gdelta_prep");
}

// The convolution's last taps - 1 inputs go into the state: by the block of a head's first value channels, the
// head's value channels, and with the first head of a group its q and k.
__device__ __forceinline__ void gd_keep_inputs(const float* __restrict__ proj, size_t ldp, float* __restrict__ tail, int taps,
                                               int t0, int n, int h, int gk, int H, int G, int D, int E) {
    if (taps <= 1) return;
    const int C = 2 * G * D + H * E;
    const int own = (h % (H / G) == 0) ? 2 * D : 0;
    for (int x = threadIdx.x; x < E + own; x += blockDim.x) {
        const int c = x < E ? 2 * G * D + h * E + x : (x - E < D ? gk * D + x - E : (G + gk) * D + x - E - D);
        for (int i = 0; i < taps - 1; ++i) {            // ascending: what is read lies behind what was written
            const int src = n - (taps - 1) + i;
            tail[(size_t)i * C + c] = src >= 0 ? proj[(size_t)(t0 + src) * ldp + c] : tail[(size_t)(i + n) * C + c];
        }
    }
}

// One token of one value channel, on the row of sixteen lanes that shares the channel; lane s holds the key
// channels s, s + 16, ... of S, k and q.  The same additions in the same order wherever it is used, so that a
// sequence gives the same bits however it is cut into steps.
template <int KPL>
__device__ __forceinline__ float gd_token(float (&S)[KPL], const float (&kk)[KPL], const float (&qq)[KPL], float v, float beta,
                                          float g) {
    float a = 0.f;
#pragma unroll
    for (int m = 0; m < KPL; ++m) a = fmaf(S[m], kk[m], a);
    a = row16_sum(a);
    const float u = beta * (v - g * a);
    float b = 0.f;
#pragma unroll
    for (int m = 0; m < KPL; ++m) {
        S[m] = fmaf(kk[m], u, g * S[m]);
        b = fmaf(S[m], qq[m], b);
    }
    return row16_sum(b);
}

// For steps in which every request brings a few tokens (decoding): no LDS and no barrier.  A row of sixteen lanes
// shares a value channel as above, but lane s takes the key channels s, s + 16, ...: a load or store of the state
// is sixteen neighbouring floats a row, and k and q come straight from the prepared rows.
template <int KPL>
__global__ __launch_bounds__(256) void gdelta_recurrence_few_kernel(
    const float* __restrict__ pre, const float* __restrict__ proj, size_t ldp, float* __restrict__ state, size_t state_row,
    size_t tail_off, int taps, const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ state_slots,
    float* __restrict__ o, int H, int G, int D, int E) {
    const int h = blockIdx.y, r = blockIdx.z, j0 = blockIdx.x * 16;
    const int tid = threadIdx.x, s = tid & 15, j = j0 + (tid >> 4), jc = min(j, E - 1);
    const int C = 2 * G * D + H * E;
    const size_t ldq = (size_t)C + 2 * H;
    const int gk = h / (H / G);
    const int t0 = cu_tokens[r], n = cu_tokens[r + 1] - t0;
    float* srow = state + (size_t)state_slots[r] * state_row;
    float* sp = srow + ((size_t)h * E + jc) * D + s;
    const bool row_live = j < E;
    float S[KPL];
#pragma unroll
    for (int m = 0; m < KPL; ++m) S[m] = (row_live && s + 16 * m < D) ? sp[16 * m] : 0.f;
    for (int t = 0; t < n; ++t) {
        const float* p = pre + (size_t)(t0 + t) * ldq;
        const float* pk = p + (size_t)(G + gk) * D + s;
        const float* pq = p + (size_t)gk * D + s;
        float kk[KPL], qq[KPL];
#pragma unroll
        for (int m = 0; m < KPL; ++m) {
            const bool in = s + 16 * m < D;
            kk[m] = in ? pk[16 * m] : 0.f;
            qq[m] = in ? pq[16 * m] : 0.f;
        }
        const float v = p[2 * (size_t)G * D + (size_t)h * E + jc], beta = p[C + h], g = p[C + H + h];
        const float b = gd_token<KPL>(S, kk, qq, v, beta, g);
        if (s == 0 && row_live) o[(size_t)(t0 + t) * H * E + (size_t)h * E + j] = b;
    }
    if (row_live) {
#pragma unroll
        for (int m = 0; m < KPL; ++m)
            if (s + 16 * m < D) sp[16 * m] = S[m];
    }
    if (blockIdx.x == 0) gd_keep_inputs(proj, ldp, srow + tail_off, taps, t0, n, h, gk, H, G, D, E);
}

// Block: sixteen value channels of one head of one request; a row of sixteen lanes shares a value channel, each
// lane the KPL key channels s, s + 16, ... of it (dim <= 16 KPL; the channels past dim are zero; in LDS a lane's
// channels of k and of q lie side by side).  The tokens of the portion pass in
// chunks of sixteen (eight for the widest heads): a chunk's k, q, its sixteen v, beta and decay are fetched into
// registers while the chunk before is worked through from LDS, so that no token waits for memory; the waves meet
// at the chunks' borders only.  Per token a lane does 4 KPL multiply-adds and two sums over its row:
//   a = S^T k (of the state before the token);   u = beta (v - g a);   S <- g S + k u;   o = S^T q.
// Only S runs from token to token; the read-out hangs off it, so with the loop unrolled by four a token's
// read-out, its store and the LDS reads of the tokens after it fill the waits of the next token's sum.
template <int KPL>
__global__ __launch_bounds__(256) void gdelta_recurrence_kernel(
    const float* __restrict__ pre, const float* __restrict__ proj, size_t ldp, float* __restrict__ state, size_t state_row,
    size_t tail_off, int taps, const int32_t* __restrict__ cu_tokens, const int32_t* __restrict__ state_slots,
    float* __restrict__ o, int H, int G, int D, int E) {
    constexpr int DP = 16 * KPL;
    constexpr int GD_CHUNK = KPL >= 16 ? 8 : 16;           // (two chunks of the widest heads fill LDS otherwise)
    constexpr int ROWW = 2 * DP + 20;                      // k, q, sixteen v, beta, decay of a token; rows of 16 bytes
    constexpr int NLD = (GD_CHUNK * ROWW + 255) / 256;
    constexpr int VEC = KPL % 4 == 0 ? 4 : (KPL % 2 == 0 ? 2 : 1);
    __shared__ __attribute__((aligned(16))) float lds[2][GD_CHUNK * ROWW];
    const int h = blockIdx.y, r = blockIdx.z, j0 = blockIdx.x * 16;
    const int tid = threadIdx.x, s = tid & 15, j = j0 + (tid >> 4);
    const int C = 2 * G * D + H * E;
    const size_t ldq = (size_t)C + 2 * H;
    const int gk = h / (H / G);
    const int t0 = cu_tokens[r], n = cu_tokens[r + 1] - t0;
    if (n <= 0) return;                                    // (the whole block: a request without tokens changes nothing)
    float* srow = state + (size_t)state_slots[r] * state_row;
    float S[KPL];
    float* sp = srow + ((size_t)h * E + min(j, E - 1)) * D + s;
#pragma unroll
    for (int m = 0; m < KPL; ++m) S[m] = (j < E && s + 16 * m < D) ? sp[16 * m] : 0.f;

    // (every element has one load at an address chosen without branches, so that the loads of a chunk are all in
    // flight together; what lies past the portion, dim or vdim reads the row's first element and is stored as zero.
    // Where an element comes from and where it goes in LDS does not change from chunk to chunk: found once.)
    float regs[NLD];
    unsigned rel[NLD], live = 0, cols = 0;
    int dst[NLD], tks[NLD];
#pragma unroll
    for (int x = 0; x < NLD; ++x) {
        const int e = x * 256 + tid;
        const int tk = e / ROWW, col = e - tk * ROWW;
        const int ck = col, cq = col - DP, cv = col - 2 * DP, cb = col - 2 * DP - 16;
        const bool isk = col < DP, isq = !isk && col < 2 * DP, isv = cv >= 0 && cv < 16, isb = cb >= 0 && cb < 2;
        const bool ok = tk < GD_CHUNK && ((isk && ck < D) || (isq && cq < D) || (isv && j0 + cv < E) || isb);
        const size_t at = isk ? (size_t)(G + gk) * D + ck
                        : isq ? (size_t)gk * D + cq
                        : isv ? 2 * (size_t)G * D + (size_t)h * E + j0 + cv
                              : (size_t)C + (size_t)cb * H + h;
        rel[x] = ok ? (unsigned)((size_t)tk * ldq + at) : 0u;
        cols |= ok ? 1u << x : 0u;
        tks[x] = tk;
        const int d = col < DP ? col : col - DP;                           // key channel d: lane d % 16, its place d / 16
        dst[x] = e < GD_CHUNK * ROWW ? tk * ROWW + (col < 2 * DP ? col - d + (d & 15) * KPL + (d >> 4) : col) : -1;
    }
    auto fetch = [&](int first) {
        const float* base = pre + (size_t)(t0 + first) * ldq;
        live = 0;
#pragma unroll
        for (int x = 0; x < NLD; ++x) {
            const bool ok = (cols >> x & 1u) && first + tks[x] < n;
            regs[x] = base[ok ? rel[x] : 0u];
            live |= ok ? 1u << x : 0u;
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int x = 0; x < NLD; ++x)
            if (dst[x] >= 0) lds[buf][dst[x]] = (live >> x & 1u) ? regs[x] : 0.f;
    };
    // a lane's KPL channels of a row of LDS, in reads of sixteen bytes where KPL allows
    auto take = [&](const float* p, float* dst) {
        if constexpr (VEC == 4) {
#pragma unroll
            for (int m = 0; m < KPL; m += 4) {
                const float4 x = *reinterpret_cast<const float4*>(p + m);
                dst[m] = x.x; dst[m + 1] = x.y; dst[m + 2] = x.z; dst[m + 3] = x.w;
            }
        } else if constexpr (VEC == 2) {
#pragma unroll
            for (int m = 0; m < KPL; m += 2) {
                const float2 x = *reinterpret_cast<const float2*>(p + m);
                dst[m] = x.x; dst[m + 1] = x.y;
            }
        } else {
#pragma unroll
            for (int m = 0; m < KPL; ++m) dst[m] = p[m];
        }
    };
    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    const bool writer = s == 0 && j < E;
    for (int first = 0; first < n; first += GD_CHUNK) {
        const bool more = first + GD_CHUNK < n;
        if (more) fetch(first + GD_CHUNK);
        const int cnt = min(GD_CHUNK, n - first);
        float* orow = o + (size_t)(t0 + first) * H * E + (size_t)h * E + min(j, E - 1);
#pragma unroll 4
        for (int tk = 0; tk < cnt; ++tk) {
            const float* L = lds[buf] + tk * ROWW;
            float kk[KPL], qq[KPL];
            take(L + s * KPL, kk);
            take(L + DP + s * KPL, qq);
            const float v = L[2 * DP + (tid >> 4)];
            const float2 bg = *reinterpret_cast<const float2*>(L + 2 * DP + 16);
            const float b = gd_token<KPL>(S, kk, qq, v, bg.x, bg.y);
            if (writer) orow[(size_t)tk * H * E] = b;
        }
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
    if (j < E) {
#pragma unroll
        for (int m = 0; m < KPL; ++m)
            if (s + 16 * m < D) sp[16 * m] = S[m];
    }
    if (blockIdx.x == 0) gd_keep_inputs(proj, ldp, srow + tail_off, taps, t0, n, h, gk, H, G, D, E);
}

TFF_API int tff_gdelta_recurrence(const float* pre, const float* proj, size_t ldp, float* state, size_t state_row,
                                  size_t tail_off, int taps, const int32_t* cu_tokens, const int32_t* state_slots, float* o,
                                  int R, int H, int G, int D, int E, int max_tokens, tff_stream_t stream) {
    TFF_REQUIRE(pre && proj && state && cu_tokens && state_slots && o, "gdelta_recurrence: null pointer");
    TFF_REQUIRE(R >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && D <= 256 && E > 0 && taps >= 1 && taps <= GD_MAX_TAPS,
                "gdelta_recurrence: bad sizes heads=%d kv_heads=%d dim=%d vdim=%d taps=%d (dim up to 256, taps up to %d)", H, G, D,
                E, taps, GD_MAX_TAPS);
    const size_t C = 2 * (size_t)G * D + (size_t)H * E;
    TFF_REQUIRE(ldp >= C + 2 * (size_t)H && (size_t)H * E * D <= tail_off && tail_off + (size_t)(taps - 1) * C <= state_row,
                "gdelta_recurrence: rows of %zu or state rows of %zu are too short", ldp, state_row);
    TFF_REQUIRE(H <= 65535 && R <= 65535, "gdelta_recurrence: too many heads or requests");
    TFF_REQUIRE((C + 2 * (size_t)H) * 17 < ((size_t)1 << 31), "gdelta_recurrence: rows of %zu channels are too long", C);
    if (R == 0) return 0;
    const dim3 grid((E + 15) / 16, H, R);
    hipStream_t s = (hipStream_t)stream;
    // (a request's tokens go one after the other: up to GD_FEW of them need no staging through LDS)
#define GD_LAUNCH(KPL)                                                                                                     \
    do {                                                                                                                   \
        if (max_tokens > 0 && max_tokens <= GD_FEW)                                                                        \
            gdelta_recurrence_few_kernel<KPL><<<grid, 256, 0, s>>>(pre, proj, ldp, state, state_row, tail_off, taps,        \
                                                                   cu_tokens, state_slots, o, H, G, D, E);                 \
        else                                                                                                               \
            gdelta_recurrence_kernel<KPL><<<grid, 256, 0, s>>>(pre, proj, ldp, state, state_row, tail_off, taps, cu_tokens, \
                                                               state_slots, o, H, G, D, E);                                \
    } while (0)
    if (D <= 16) GD_LAUNCH(1);
    else if (D <= 32) GD_LAUNCH(2);
    else if (D <= 64) GD_LAUNCH(4);
    else if (D <= 128) GD_LAUNCH(8);
    else GD_LAUNCH(16);
#undef GD_LAUNCH
    return tff_check_launch("gdelta_recurrence");
}

// One wave per (token, head): the head's E channels of o are divided by their root mean square, multiplied by
// w[channel] (one weight for all heads) and by silu(gate), and go to out[t * out_row + h * E + e].
template <typename TO>
__global__ __launch_bounds__(256) void head_norm_silu_gate_kernel(const float* __restrict__ o, const float* __restrict__ g,
                                                                  size_t g_row, const float* __restrict__ w, float eps,
                                                                  float scale, TO* __restrict__ out, size_t out_row,
                                                                  int pairs, int H, int E) {
    const int id = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (id >= pairs) return;
    const int t = id / H, h = id % H;
    const float* orow = o + ((size_t)t * H + h) * E;
    float ss = 0.f;
    for (int e = lane; e < E; e += 64) ss = fmaf(orow[e], orow[e], ss);
    ss = wave_sum(ss);
    const float rr = scale / sqrtf(ss / (float)E + eps);
    const float* grow = g + (size_t)t * g_row + (size_t)h * E;
    for (int e = lane; e < E; e += 64)
        out[(size_t)t * out_row + (size_t)h * E + e] = from_f32<TO>(orow[e] * rr * w[e] * gd_silu(grow[e]));
}

TFF_API int tff_head_norm_silu_gate(const float* o, const float* g, size_t g_row, const float* w, float eps, float scale,
                                    void* out, size_t out_row, int T, int H, int E, int out_dtype, tff_stream_t stream) {
    TFF_REQUIRE(o && g && w && out, "head_norm_silu_gate: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && E > 0 && g_row >= (size_t)H * E && out_row >= (size_t)H * E, "head_norm_silu_gate: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int pairs = T * H;
    if (out_dtype == TFF_F32)
        head_norm_silu_gate_kernel<float><<<(pairs + 3) / 4, 256, 0, s>>>(o, g, g_row, w, eps, scale, (float*)out, out_row, pairs, H, E);
    else if (out_dtype == TFF_BF16)
        head_norm_silu_gate_kernel<bf16_t><<<(pairs + 3) / 4, 256, 0, s>>>(o, g, g_row, w, eps, scale, (bf16_t*)out, out_row, pairs, H, E);
    else
        return tff_fail("head_norm_silu_gate: unknown dtype %d", out_dtype);
    return tff_check_launch("head_norm_silu_gate");
}

// out[t * out_row + h * E + e] = o[t * o_row + h * o_head + e] * sigmoid(g[t * g_row + h * E + e]) * scale
template <typename T>
__global__ __launch_bounds__(256) void sigmoid_gate_heads_kernel(const T* __restrict__ o, size_t o_row, int o_head,
                                                                 const T* __restrict__ g, size_t g_row, float scale,
                                                                 T* __restrict__ out, size_t out_row, int HE, int E,
                                                                 size_t count) {
    const size_t id = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= count) return;
    const size_t t = id / HE;
    const int c = (int)(id - t * HE), h = c / E, e = c - h * E;
    const float gz = to_f32(g[t * g_row + c]);
    out[t * out_row + c] = from_f32<T>(to_f32(o[t * o_row + (size_t)h * o_head + e]) * (scale / (1.0f + expf(-gz))));
}

TFF_API int tff_sigmoid_gate_heads(const void* o, size_t o_row, int o_head, const void* g, size_t g_row, float scale, void* out,
                                   size_t out_row, int T, int H, int E, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(o && g && out, "sigmoid_gate_heads: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && E > 0 && o_head >= E && o_row >= (size_t)H * o_head && g_row >= (size_t)H * E &&
                out_row >= (size_t)H * E, "sigmoid_gate_heads: bad sizes");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const size_t count = (size_t)T * H * E;
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (dtype == TFF_F32)
        sigmoid_gate_heads_kernel<float><<<blocks, 256, 0, s>>>((const float*)o, o_row, o_head, (const float*)g, g_row, scale,
                                                                (float*)out, out_row, H * E, E, count);
    else if (dtype == TFF_BF16)
        sigmoid_gate_heads_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)o, o_row, o_head, (const bf16_t*)g, g_row, scale,
                                                                 (bf16_t*)out, out_row, H * E, E, count);
    else
        return tff_fail("sigmoid_gate_heads: unknown dtype %d", dtype);
    return tff_check_launch("sigmoid_gate_heads");
}
