// A feed-forward made of many small experts of which every token uses a few.
//
// tff_route_topk:   z = Wr h in float32 (or given: a product that ran before), s = sigmoid(z); the `top` experts with the largest
//                   s + bias are chosen (the lowest index among equals), their weights are
//                   s / (sum of the chosen s + 1e-20): the bias moves the choice only.  With `softmax`,
//                   s = softmax(z) over all experts and the weights are the chosen s as they are.
// tff_experts_gate_up: for every (token, chosen expert): g = min(Wg h, limit),
//                   u = clamp(Wu h, -limit, limit), y = g * sigmoid(act_alpha * g) * (u + up_offset)
//                   (limit = infinity, act_alpha = 1, up_offset = 0: silu(g) * u).
// tff_experts_down: out[t] = sum over the token's experts, in the order they were chosen, of
//                   weight * (Wd y), float32.
//
// The two expert kernels give every (token, expert) pair waves of its own that stream the
// expert's rows once: what a step of few tokens is bound by.  Each output element is one
// wave's dot product in a fixed order of k, so a token's result does not depend on what else
// the step holds.  Expert weights lie [experts, out, in], row-major, rows ldw elements apart (ldw >= in:
// rows a power of two of bytes apart all come through one memory channel, so the loader puts a
// little room behind each).
#include "common.h"
#include "tffinfer_kernels.h"

// dot product of two rows of K elements by one wave (lanes stride through k, then a tree)
template <typename TA, typename TB>
__device__ __forceinline__ float wave_dot(const TA* __restrict__ a, const TB* __restrict__ b, int K, int lane) {
    float acc = 0.f;
    for (int k = lane; k < K; k += 64) acc = fmaf(to_f32(a[k]), to_f32(b[k]), acc);
    return wave_sum(acc);
}
// both rows bfloat16, K a multiple of 8 and both 16-byte aligned: eight elements a load
__device__ __forceinline__ float wave_dot8(const bf16_t* __restrict__ a, const bf16_t* __restrict__ b, int K, int lane) {
    float acc = 0.f;
    for (int k = lane * 8; k < K; k += 512) {
        union { uint4 u; bf16_t h[8]; } x, y;
        x.u = *reinterpret_cast<const uint4*>(a + k);
        y.u = *reinterpret_cast<const uint4*>(b + k);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc = fmaf((float)x.h[j], (float)y.h[j], acc);
    }
    return wave_sum(acc);
}
template <typename T>
__device__ __forceinline__ float row_dot(const T* a, const T* b, int K, int lane, bool vec) {
    return wave_dot(a, b, K, lane);
}
template <>
__device__ __forceinline__ float row_dot<bf16_t>(const bf16_t* a, const bf16_t* b, int K, int lane, bool vec) {
    return vec ? wave_dot8(a, b, K, lane) : wave_dot(a, b, K, lane);
}

#define RT_MAX_E 1024

// One block of RT_WAVES waves per token.  logits != null: z is given (a product that ran before);
// else the waves compute it, each its share of the experts, 16 bytes a lane and load.
#define RT_WAVES 8

template <typename T>
__global__ __launch_bounds__(64 * RT_WAVES) void route_topk_kernel(const T* __restrict__ h, int h_row,
                                                                   const float* __restrict__ Wr,
                                                                   const float* __restrict__ logits,
                                                                   const float* __restrict__ bias, int width, int E,
                                                                   int top, int softmax, int32_t* __restrict__ idx,
                                                                   float* __restrict__ wts) {
    __shared__ float s_all[RT_MAX_E];
    __shared__ float c_all[RT_MAX_E];
    __shared__ int chosen[64];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    if (logits) {
        for (int e = threadIdx.x; e < E; e += blockDim.x) s_all[e] = logits[(size_t)t * E + e];
    } else {
        const T* hr = h + (size_t)t * h_row;
        for (int e = wv; e < E; e += RT_WAVES) {
            const float z = wave_dot(hr, Wr + (size_t)e * width, width, lane);
            if (lane == 0) s_all[e] = z;
        }
    }
    __syncthreads();
    if (wv > 0) return;
    // (one wave from here on: LDS works through its accesses in order)
    if (softmax == 1) {
        // s = exp(z - max) / sum over all experts, the sum in the order of the lanes' strides and a tree
        float mx = -INFINITY;
        for (int e = lane; e < E; e += 64) mx = fmaxf(mx, s_all[e]);
        mx = wave_max(mx);
        float den = 0.f;
        for (int e = lane; e < E; e += 64) {
            const float x = expf(s_all[e] - mx);
            s_all[e] = x;
            den += x;
        }
        den = wave_sum(den);
        for (int e = lane; e < E; e += 64) {
            const float s = s_all[e] / den;
            s_all[e] = s;
            c_all[e] = s + (bias ? bias[e] : 0.f);
        }
    } else {
        for (int e = lane; e < E; e += 64) {
            const float s = 1.0f / (1.0f + expf(-s_all[e]));
            s_all[e] = s;
            c_all[e] = s + (bias ? bias[e] : 0.f);
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
    __builtin_amdgcn_wave_barrier();
    float sum = 0.f;
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
        for (int e = lane; e < E; e += 64) {
            const float c = c_all[e];
            if (c > best) { best = c; bi = e; }      // (ascending e: the first of equals stays)
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oi = __shfl_xor(bi, o, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        // (one wave from here on: LDS works through its accesses in order)
        if (lane == 0) {
            idx[(size_t)t * top + k] = bi;
            chosen[k] = bi;
            c_all[bi] = -INFINITY;
        }
        sum += s_all[bi];
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
        __builtin_amdgcn_wave_barrier();
    }
    const float inv = softmax ? 1.0f : 1.0f / (sum + 1e-20f);      // (mode 2: sigmoid scores as they are)
    if (lane < top) wts[(size_t)t * top + lane] = s_all[chosen[lane]] * inv;
}

TFF_API int tff_route_topk(const void* h, int h_row, const float* Wr, const float* logits, const float* bias, int T,
                           int width, int E, int top, int softmax, int32_t* idx, float* wts, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(idx && wts && (logits || (h && Wr)), "route_topk: null pointer");
    TFF_REQUIRE(T >= 0 && (logits || (width > 0 && h_row >= width)), "route_topk: bad sizes T=%d width=%d row=%d", T, width, h_row);
    TFF_REQUIRE(E > 0 && E <= RT_MAX_E && top > 0 && top <= E && top <= 64,
                "route_topk: %d of %d experts (up to 64 of up to %d)", top, E, RT_MAX_E);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == TFF_F32)
        route_topk_kernel<float><<<T, 64 * RT_WAVES, 0, s>>>((const float*)h, h_row, Wr, logits, bias, width, E, top, softmax, idx, wts);
    else if (dtype == TFF_BF16)
        route_topk_kernel<bf16_t><<<T, 64 * RT_WAVES, 0, s>>>((const bf16_t*)h, h_row, Wr, logits, bias, width, E, top, softmax, idx, wts);
    else
        return tff_fail("route_topk: unknown dtype %d", dtype);
    return tff_check_launch("route_topk");
}

// Experts by a table over the token ids instead of a router: idx[t, k] = table[ids[t], k], each with the weight
// 1 / top.  An id or an expert outside its range is brought into it (a launch never reads outside a table).
__global__ __launch_bounds__(256) void route_by_table_kernel(const int32_t* __restrict__ table, const int32_t* __restrict__ ids,
                                                             int pairs, int V, int top, int E, int32_t* __restrict__ idx,
                                                             float* __restrict__ wts) {
    const int p = blockIdx.x * 256 + threadIdx.x;
    if (p >= pairs) return;
    const int t = p / top, k = p - t * top;
    const int id = min(max(ids[t], 0), V - 1);
    idx[p] = min(max(table[(size_t)id * top + k], 0), E - 1);
    wts[p] = 1.0f / (float)top;
}

TFF_API int tff_route_by_table(const int32_t* table, const int32_t* ids, int T, int V, int top, int E, int32_t* idx,
                               float* wts, tff_stream_t stream) {
    TFF_REQUIRE(table && ids && idx && wts, "route_by_table: null pointer");
    TFF_REQUIRE(T >= 0 && V > 0 && top > 0 && E > 0, "route_by_table: bad sizes T=%d V=%d top=%d E=%d", T, V, top, E);
    if (T == 0) return 0;
    route_by_table_kernel<<<(T * top + 255) / 256, 256, 0, (hipStream_t)stream>>>(table, ids, T * top, V, top, E, idx, wts);
    return tff_check_launch("route_by_table");
}

#define EX_WAVES 4
#define EX_PER_WAVE 8      // outputs a wave works through

template <typename T>
__global__ __launch_bounds__(64 * EX_WAVES) void experts_gate_up_kernel(
    const T* __restrict__ h, int h_row, const T* __restrict__ Wg, const T* __restrict__ Wu,
    const int32_t* __restrict__ idx, int top, int width, int ff, int ldw, float limit, float act_alpha, float up_offset,
    const float* __restrict__ in_wts, T* __restrict__ y) {
    // Wg null: experts without a gate, y = max(Wu h, 0)^2.  in_wts: the pair's weight multiplies what goes into the
    // expert, W (w h) = w (W h): both products times w before clamps and activation.
    const int pair = blockIdx.x;                  // token * top + k
    const int t = pair / top;
    const int e = idx[pair];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const T* hr = h + (size_t)t * h_row;
    const T* wg = Wg ? Wg + (size_t)e * ff * ldw : nullptr;
    const T* wu = Wu + (size_t)e * ff * ldw;
    const bool vec = sizeof(T) == 2 && width % 8 == 0 && ldw % 8 == 0 && h_row % 8 == 0 && ((uintptr_t)h % 16) == 0 &&
                     ((uintptr_t)Wg % 16) == 0 && ((uintptr_t)Wu % 16) == 0;
    const float win = in_wts ? in_wts[pair] : 1.0f;
    const int f0 = (blockIdx.y * EX_WAVES + wv) * EX_PER_WAVE;
    for (int f = f0; f < min(ff, f0 + EX_PER_WAVE); ++f) {
        float u = row_dot<T>(hr, wu + (size_t)f * ldw, width, lane, vec) * win;
        if (!wg) {
            if (lane == 0) {
                u = fmaxf(u, 0.f);
                y[(size_t)pair * ff + f] = from_f32<T>(u * u);
            }
            continue;
        }
        float g = row_dot<T>(hr, wg + (size_t)f * ldw, width, lane, vec) * win;
        if (lane == 0) {
            g = fminf(g, limit);
            u = fminf(fmaxf(u, -limit), limit);
            const float a = g * (1.0f / (1.0f + expf(-act_alpha * g))) * (u + up_offset);
            y[(size_t)pair * ff + f] = from_f32<T>(a);
        }
    }
}

template <typename T>
__global__ __launch_bounds__(64 * EX_WAVES) void experts_down_kernel(
    const T* __restrict__ y, const T* __restrict__ Wd, const int32_t* __restrict__ idx, const float* __restrict__ wts,
    int top, int width, int ff, int ldw, float* __restrict__ out) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const bool vec = sizeof(T) == 2 && ff % 8 == 0 && ldw % 8 == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)Wd % 16) == 0;
    const int n0 = (blockIdx.y * EX_WAVES + wv) * EX_PER_WAVE;
    for (int n = n0; n < min(width, n0 + EX_PER_WAVE); ++n) {
        float acc = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = idx[(size_t)t * top + k];
            const float d = row_dot<T>(y + ((size_t)t * top + k) * ff, Wd + ((size_t)e * width + n) * ldw, ff, lane, vec);
            acc = fmaf(wts ? wts[(size_t)t * top + k] : 1.0f, d, acc);
        }
        if (lane == 0) out[(size_t)t * width + n] = acc;
    }
}

TFF_API int tff_experts_gate_up(const void* h, int h_row, const void* Wg, const void* Wu, const int32_t* idx, int T,
                                int top, int E, int width, int ff, int ldw, float limit, float act_alpha, float up_offset,
                                const float* in_wts, void* y,
                                int dtype, tff_stream_t stream) {
    TFF_REQUIRE(h && Wu && idx && y, "experts_gate_up: null pointer");
    TFF_REQUIRE(T >= 0 && top > 0 && E > 0 && width > 0 && ff > 0 && h_row >= width && ldw >= width,
                "experts_gate_up: bad sizes T=%d top=%d width=%d ff=%d", T, top, width, ff);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(T * top, (ff + EX_WAVES * EX_PER_WAVE - 1) / (EX_WAVES * EX_PER_WAVE));
    TFF_REQUIRE(grid.y <= 65535, "experts_gate_up: too many outputs");
    if (dtype == TFF_F32)
        experts_gate_up_kernel<float><<<grid, 64 * EX_WAVES, 0, s>>>((const float*)h, h_row, (const float*)Wg, (const float*)Wu,
                                                                    idx, top, width, ff, ldw, limit, act_alpha, up_offset, in_wts, (float*)y);
    else if (dtype == TFF_BF16)
        experts_gate_up_kernel<bf16_t><<<grid, 64 * EX_WAVES, 0, s>>>((const bf16_t*)h, h_row, (const bf16_t*)Wg,
                                                                     (const bf16_t*)Wu, idx, top, width, ff, ldw, limit,
                                                                     act_alpha, up_offset, in_wts, (bf16_t*)y);
    else
        return tff_fail("experts_gate_up: unknown dtype %d", dtype);
    return tff_check_launch("experts_gate_up");
}

TFF_API int tff_experts_down(const void* y, const void* Wd, const int32_t* idx, const float* wts, int T, int top, int E,
                             int width, int ff, int ldw, float* out, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(y && Wd && idx && out, "experts_down: null pointer");      // (wts null: every pair counts 1)
    TFF_REQUIRE(T >= 0 && top > 0 && E > 0 && width > 0 && ff > 0 && ldw >= ff, "experts_down: bad sizes T=%d top=%d width=%d ff=%d",
                T, top, width, ff);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const dim3 grid(T, (width + EX_WAVES * EX_PER_WAVE - 1) / (EX_WAVES * EX_PER_WAVE));
    TFF_REQUIRE(grid.y <= 65535, "experts_down: too many outputs");
    if (dtype == TFF_F32)
        experts_down_kernel<float><<<grid, 64 * EX_WAVES, 0, s>>>((const float*)y, (const float*)Wd, idx, wts, top, width, ff, ldw, out);
    else if (dtype == TFF_BF16)
        experts_down_kernel<bf16_t><<<grid, 64 * EX_WAVES, 0, s>>>((const bf16_t*)y, (const bf16_t*)Wd, idx, wts, top, width, ff, ldw, out);
    else
        return tff_fail("experts_down: unknown dtype %d", dtype);
    return tff_check_launch("experts_down");
}

// ------------------------------------------------------------- many tokens: by expert ---
// With many tokens a step the (token, expert) pairs are dealt to their experts first: every
// expert's pairs fill tiles of `rows` pairs (64, or 128 where the experts have a few hundred pairs
// each; an expert's last tile is padded), so that a tile's rows share the expert's matrices and the
// products run on the matrix cores.  A pair's row is computed from the pair alone, k ascending,
// whatever tile and place it lands in: the result does not depend on what else the step holds, nor
// on the order the pairs were dealt in.
//
// experts_sort_kernel:  tile_expert[tile], tile_rows[tile * rows + i] = pair (token * top + k) or -1,
//                       num_tiles[0]; one block.  At most pairs / rows + E tiles.
// experts_tiles_kernel: the two products per tile.  The down product writes
//                       out[k][t][:] = wts[t][k] * Wd y: `top` planes that the norm after the
//                       feed-forward adds up in the order of k.

__global__ __launch_bounds__(1024) void experts_sort_kernel(const int32_t* __restrict__ idx, int pairs, int E,
                                                            int rows, int32_t* __restrict__ tile_expert,
                                                            int32_t* __restrict__ tile_rows,
                                                            int32_t* __restrict__ num_tiles) {
    __shared__ int count[RT_MAX_E];
    __shared__ int first[RT_MAX_E + 1];     // an expert's first tile
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += blockDim.x) count[e] = 0;
    __syncthreads();
    for (int p = tid; p < pairs; p += blockDim.x) atomicAdd(&count[idx[p]], 1);
    __syncthreads();
    if (tid == 0) {
        int t = 0;
        for (int e = 0; e < E; ++e) {
            first[e] = t;
            t += (count[e] + rows - 1) / rows;
        }
        first[E] = t;
        num_tiles[0] = t;
    }
    __syncthreads();
    const int tiles = first[E];
    for (int e = tid; e < E; e += blockDim.x) {
        for (int t = first[e]; t < first[e + 1]; ++t) tile_expert[t] = e;
        count[e] = 0;
    }
    for (int i = tid; i < tiles * rows; i += blockDim.x) tile_rows[i] = -1;
    __syncthreads();
    for (int p = tid; p < pairs; p += blockDim.x) {
        const int e = idx[p];
        const int at = atomicAdd(&count[e], 1);
        tile_rows[first[e] * rows + at] = p;
    }
}

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 ex_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float ex_floatx4;

__device__ __forceinline__ ex_bf16x8 ex_load8(const bf16_t* p, bool ok) {
    union { uint4 u; ex_bf16x8 v; } x;
    x.u = ok ? *reinterpret_cast<const uint4*>(p) : make_uint4(0, 0, 0, 0);
    return x.v;
}

// One kernel for both products.  Block: one tile of 64 or 128 pairs x 128 weight rows, four waves side by
// side, each all pairs x 32 weight rows (eight or sixteen accumulators).  GATE_UP: a wave's 32 weight rows
// are 16 outputs of the gate and the same 16 of the up projection; else 32 outputs of the down
// projection.  K goes in steps of 64.  The pairs' rows, which all four waves need, pass through LDS
// (global -> registers while the step before is computed, then registers -> LDS; a fragment of 16
// rows x 32 k lies there as a wave reads it, lane l's eight elements at l * 16 bytes); a wave's own
// weight rows go straight from memory into its MFMA operands, one step ahead: LDS bandwidth is what
// bounds a block of few waves, and the weight is two thirds of the operands.
// C[w][pair] += W[w][k] a[pair][k]: lane (pair = lane & 15, kg = lane >> 4) ends up with weight rows
// kg * 4 .. + 3 of its pair.  k ascends for every pair alike, whatever tile and place the pair was
// dealt to.
#define EXT_KSTEP 64

// MODE 0: the down product; 1: gate and up; 2: up alone, y = max(Wu h, 0)^2 (a wave's 32 weight rows are 32 outputs).
template <int MODE, int AFR>
__global__ __launch_bounds__(256) void experts_tiles_kernel(
    const bf16_t* __restrict__ a_rows, int a_row, const bf16_t* __restrict__ W0, const bf16_t* __restrict__ W1,
    const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_rows,
    const int32_t* __restrict__ num_tiles, const float* __restrict__ wts, int T, int top, int K, int N,
    float limit, float act_alpha, float up_offset, bf16_t* __restrict__ y, float* __restrict__ out, int max_tiles, int col_blocks,
    int ldw, int weight_input) {
    // weight_input: a pair's weight multiplies what goes into its expert (both first products, before clamps
    // and activation: W (w h) = w (W h)) and the second product counts 1
    constexpr bool GATE_UP = MODE == 1;
    constexpr int ROWS = AFR * 16;       // pairs of a tile: 64, or 128 where the experts have many pairs each
    __shared__ __attribute__((aligned(16))) bf16_t lds[2 * AFR * 512];      // two sub-steps of AFR fragments
    // A tile of 64 pairs gives a weight element 128 flops a read: the tiles of one expert must meet
    // their weight rows in a cache, or the products run at what memory gives.  Blocks go to the
    // eight XCDs in turn by their number, each XCD with an L2 of its own; so block L works on
    // column block (L / 8 / max_tiles) * 8 + L % 8 and tile L / 8 % max_tiles: one XCD sees all
    // tiles of a column block one after the other, an expert's tiles next to each other.
    const int L = blockIdx.x, q = L >> 3;
    const int tile = q % max_tiles, col_block = (q / max_tiles) * 8 + (L & 7);
    if (tile >= num_tiles[0] || col_block >= col_blocks) return;
    const int tid = threadIdx.x, lane = tid & 63, wv = tid >> 6, r = lane & 15, kg = lane >> 4;
    const int e = tile_expert[tile];
    const int c0 = col_block * (GATE_UP ? 64 : 128) + wv * (GATE_UP ? 16 : 32);     // the wave's first output
    // the pairs' rows: 2 AFR fragments a step (AFR of 16 pairs, two sub-steps of 32 k), AFR / 2 a wave
    constexpr int AU = AFR / 2;
    const bf16_t* asrc[AU];
    bool aok[AU];
#pragma unroll
    for (int i = 0; i < AU; ++i) {
        const int fs = i * 4 + wv, sub = fs / AFR, frag = fs % AFR;
        const int pair = tile_rows[tile * ROWS + frag * 16 + r];
        aok[i] = pair >= 0;
        asrc[i] = a_rows + (size_t)(MODE != 0 ? max(pair, 0) / top : max(pair, 0)) * a_row + sub * 32 + kg * 8;
    }
    // the wave's weight rows: two fragments
    const bf16_t* wsrc[2];
    bool wok[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = GATE_UP ? c0 + r : c0 + j * 16 + r;
        wok[j] = n < N;
        wsrc[j] = ((GATE_UP && j == 1) ? W1 : W0) + ((size_t)e * N + min(n, N - 1)) * ldw + kg * 8;
    }
    ex_floatx4 acc[2][AFR];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int i = 0; i < AFR; ++i) acc[j][i] = ex_floatx4{0.f, 0.f, 0.f, 0.f};
    uint4 areg[AU];
    ex_bf16x8 wreg[2][2];        // [sub][fragment] of the step that is fetched
    auto fetch = [&](int k0) {
#pragma unroll
        for (int i = 0; i < AU; ++i) {
            const int sub = (i * 4 + wv) / AFR;
            const bool in = aok[i] && k0 + sub * 32 + kg * 8 < K;
            areg[i] = in ? *reinterpret_cast<const uint4*>(asrc[i] + k0) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
            for (int j = 0; j < 2; ++j) wreg[sub][j] = ex_load8(wsrc[j] + k0 + sub * 32, wok[j] && k0 + sub * 32 + kg * 8 < K);
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += EXT_KSTEP) {
        __syncthreads();            // the step before is read
#pragma unroll
        for (int i = 0; i < AU; ++i) *reinterpret_cast<uint4*>(lds + (size_t)(i * 4 + wv) * 512 + lane * 8) = areg[i];
        ex_bf16x8 wnow[2][2];
#pragma unroll
        for (int sub = 0; sub < 2; ++sub)
#pragma unroll
            for (int j = 0; j < 2; ++j) wnow[sub][j] = wreg[sub][j];
        __syncthreads();
        if (k0 + EXT_KSTEP < K) fetch(k0 + EXT_KSTEP);      // travels while this step is computed
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            ex_bf16x8 av[AFR];
#pragma unroll
            for (int i = 0; i < AFR; ++i)
                av[i] = *reinterpret_cast<const ex_bf16x8*>(lds + (size_t)(sub * AFR + i) * 512 + lane * 8);
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int i = 0; i < AFR; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wnow[sub][j], av[i], acc[j][i], 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < AFR; ++i) {
        const int pair = tile_rows[tile * ROWS + i * 16 + r];
        const float win = (MODE != 0 && weight_input && pair >= 0) ? wts[pair] : 1.0f;
        if (GATE_UP) {
            const float g4[4] = {acc[0][i][0], acc[0][i][1], acc[0][i][2], acc[0][i][3]};
            const float u4[4] = {acc[1][i][0], acc[1][i][1], acc[1][i][2], acc[1][i][3]};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int f = c0 + kg * 4 + c;
                if (pair >= 0 && f < N) {
                    const float gv = fminf(g4[c] * win, limit);
                    const float uv = fminf(fmaxf(u4[c] * win, -limit), limit);
                    y[(size_t)pair * N + f] = (bf16_t)(gv * (1.0f / (1.0f + expf(-act_alpha * gv))) * (uv + up_offset));
                }
            }
        } else if (MODE == 2) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float v4[4] = {acc[j][i][0], acc[j][i][1], acc[j][i][2], acc[j][i][3]};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int n = c0 + j * 16 + kg * 4 + c;
                    const float u = fmaxf(v4[c] * win, 0.f);
                    if (pair >= 0 && n < N) y[(size_t)pair * N + n] = (bf16_t)(u * u);
                }
            }
        } else {
            const int p = max(pair, 0), t = p / top, k = p - t * top;
            const float w = weight_input ? 1.0f : wts[p];
            float* o = out + ((size_t)k * T + t) * N;
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float v4[4] = {acc[j][i][0], acc[j][i][1], acc[j][i][2], acc[j][i][3]};
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int n = c0 + j * 16 + kg * 4 + c;
                    if (pair >= 0 && n < N) o[n] = w * v4[c];
                }
            }
        }
    }
}

TFF_API int tff_experts_tiles_supported(int width, int ff, int h_row) {
    return width % 8 == 0 && ff % 8 == 0 && h_row % 8 == 0;
}

// h [T, width] bfloat16; workspace: tile_expert [max_tiles], tile_rows [max_tiles * 128], num_tiles [1] (int32),
// y [T * top, ff] bfloat16; out float32 [top, T, width].  max_tiles >= T * top / 64 + E.
TFF_API int tff_experts_by_tiles(const void* h, int h_row, const void* Wg, const void* Wu, const void* Wd,
                                 const int32_t* idx, const float* wts, int T, int top, int E, int width, int ff,
                                 int ldw_in, int ldw_down, float limit, float act_alpha, float up_offset, int32_t* tile_expert,
                                 int32_t* tile_rows, int32_t* num_tiles, int max_tiles, void* y, float* out,
                                 int weight_input, tff_stream_t stream) {
    TFF_REQUIRE(h && Wu && Wd && idx && wts && tile_expert && tile_rows && num_tiles && y && out,
                "experts_by_tiles: null pointer");
    TFF_REQUIRE(T >= 0 && top > 0 && E > 0 && E <= RT_MAX_E && width > 0 && ff > 0 && h_row >= width,
                "experts_by_tiles: bad sizes T=%d top=%d E=%d width=%d ff=%d", T, top, E, width, ff);
    TFF_REQUIRE(tff_experts_tiles_supported(width, ff, h_row) && ldw_in % 8 == 0 && ldw_down % 8 == 0 && ldw_in >= width &&
                ldw_down >= ff, "experts_by_tiles: width %d, ff %d, rows of %d and the weights' rows of %d and %d must be "
                "multiples of 8", width, ff, h_row, ldw_in, ldw_down);
    TFF_REQUIRE(((uintptr_t)h % 16) == 0 && ((uintptr_t)Wg % 16) == 0 && ((uintptr_t)Wu % 16) == 0 &&
                ((uintptr_t)Wd % 16) == 0 && ((uintptr_t)y % 16) == 0, "experts_by_tiles: operands must be 16-byte aligned");
    TFF_REQUIRE((long)T * top < (1L << 31) && max_tiles <= (1 << 20) && max_tiles >= (long)T * top / 64 + E,
                "experts_by_tiles: %d tiles do not hold %d x %d pairs of %d experts", max_tiles, T, top, E);
    // tiles of 128 pairs where an expert has a few hundred on average: every weight element fetched
    // serves twice the flops, which is what bounds these products; the padding of an expert's last
    // tile costs more with fewer pairs
    const bool tall = (long)T * top >= 192L * E;
    const int rows = tall ? 128 : 64;
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    experts_sort_kernel<<<1, 1024, 0, s>>>(idx, T * top, E, rows, tile_expert, tile_rows, num_tiles);
    int rc = tff_check_launch("experts_sort");
    if (rc) return rc;
    const int cb_up = Wg ? (ff + 63) / 64 : (ff + 127) / 128, cb_down = (width + 127) / 128;
#define EXT_LAUNCH(GU, AFRV, CB, ...) experts_tiles_kernel<GU, AFRV><<<((CB) + 7) / 8 * 8 * max_tiles, 256, 0, s>>>(__VA_ARGS__)
    if (!Wg && tall)
        EXT_LAUNCH(2, 8, cb_up, (const bf16_t*)h, h_row, (const bf16_t*)Wu, nullptr, tile_expert, tile_rows,
                   num_tiles, wts, T, top, width, ff, limit, act_alpha, up_offset, (bf16_t*)y, nullptr, max_tiles, cb_up, ldw_in, weight_input);
    else if (!Wg)
        EXT_LAUNCH(2, 4, cb_up, (const bf16_t*)h, h_row, (const bf16_t*)Wu, nullptr, tile_expert, tile_rows,
                   num_tiles, wts, T, top, width, ff, limit, act_alpha, up_offset, (bf16_t*)y, nullptr, max_tiles, cb_up, ldw_in, weight_input);
    else if (tall)
        EXT_LAUNCH(1, 8, cb_up, (const bf16_t*)h, h_row, (const bf16_t*)Wg, (const bf16_t*)Wu, tile_expert, tile_rows,
                   num_tiles, wts, T, top, width, ff, limit, act_alpha, up_offset, (bf16_t*)y, nullptr, max_tiles, cb_up, ldw_in, weight_input);
    else
        EXT_LAUNCH(1, 4, cb_up, (const bf16_t*)h, h_row, (const bf16_t*)Wg, (const bf16_t*)Wu, tile_expert, tile_rows,
                   num_tiles, wts, T, top, width, ff, limit, act_alpha, up_offset, (bf16_t*)y, nullptr, max_tiles, cb_up, ldw_in, weight_input);
    rc = tff_check_launch("experts_gate_up_tiles");
    if (rc) return rc;
    if (tall)
        EXT_LAUNCH(0, 8, cb_down, (const bf16_t*)y, ff, (const bf16_t*)Wd, nullptr, tile_expert, tile_rows, num_tiles, wts,
                   T, top, ff, width, limit, act_alpha, up_offset, nullptr, out, max_tiles, cb_down, ldw_down, weight_input);
    else
        EXT_LAUNCH(0, 4, cb_down, (const bf16_t*)y, ff, (const bf16_t*)Wd, nullptr, tile_expert, tile_rows, num_tiles, wts,
                   T, top, ff, width, limit, act_alpha, up_offset, nullptr, out, max_tiles, cb_down, ldw_down, weight_input);
#undef EXT_LAUNCH
    return tff_check_launch("experts_down_tiles");
}
