// Differential attention: what stands around the paged attention kernels when every head has two
// score maps over the same values and the second map's output is subtracted from the first's.
//
// Per head h (kv head g) and map m in {0, 1}: a_m = softmax(score(q_hm . k_gm)) V_g; the head's output is
//   o = a_0 - lambda a_1,   o <- o / sqrt(mean(o^2) + eps) * out_scale,   o <- o * sigmoid(gate).
// The two maps run on the paged kernels of this library as 2 H query heads on G kv heads whose key is
// both maps' keys side by side, [k_g0 | k_g1 | 0 ..] up to the cache's head size P, with queries that
// are zero outside their own map's part, [q_h0 | 0 ..] and [0 | q_h1 | 0 ..]: a score picks its own
// map's key, query head 2 h + m reads kv head (2 h + m) / (2 H / G) = g as every grouped head does, and
// the values are stored once.
//
// tff_diff_qkv_store:  biases, rotation of both maps of q and k, the queries laid out as above, the
//                      token's key and value into its slot.
// tff_diff_combine:    the difference, the norm over the head, the gate.
#include "common.h"
#include "tffinfer_kernels.h"

struct DiffRot {
    const float* cs;     // the position's [pair][cos, sin], or null
    int dims;            // rotated elements of a map (even)
    int pairing;         // 0: (i, i + dims/2), 1: (2i, 2i+1)
};

// Element e of a map (D elements at x, bias at b or null) after the rotation.
__device__ __forceinline__ float diff_rotated(const float* __restrict__ x, const float* __restrict__ b, int e,
                                              const DiffRot r) {
    const float v = x[e] + (b ? b[e] : 0.f);
    if (!r.cs || e >= r.dims) return v;
    int i, other;
    bool first;
    if (r.pairing == 0) {
        const int half = r.dims >> 1;
        first = e < half;
        i = first ? e : e - half;
        other = first ? e + half : e - half;
    } else {
        first = !(e & 1);
        i = e >> 1;
        other = e ^ 1;
    }
    const float o = x[other] + (b ? b[other] : 0.f);
    const float c = r.cs[2 * i], s = r.cs[2 * i + 1];
    // the pair (u, w) becomes (u c - w s, w c + u s)
    return first ? fmaf(v, c, -(o * s)) : fmaf(v, c, o * s);
}

// Blocks (token, y): y < q_blocks works through DQ_HEADS query heads (head 2 h + m holds map m at elements
// m D .. m D + D - 1 and zeros elsewhere); the others are one kv head each: its key row and its value row into the
// token's slot.  A thread's elements lie DQ_THREADS apart, so no index is divided.
#define DQ_THREADS 128
#define DQ_HEADS 8

template <typename TC>
__global__ __launch_bounds__(DQ_THREADS) void diff_qkv_store_kernel(
    const float* __restrict__ proj, size_t row, const float* __restrict__ qb, const float* __restrict__ kb,
    const float* __restrict__ vb, const float* __restrict__ cos_sin, int rot_dims, int pairing, int max_pos,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, TC* __restrict__ q_out,
    TC* __restrict__ k_cache, TC* __restrict__ v_cache, int page_size, int H, int G, int D, int E, int P, int q_blocks) {
    const int t = blockIdx.x, y = blockIdx.y, tid = threadIdx.x;
    const float* x = proj + (size_t)t * row;
    const int pos = min(max(positions[t], 0), max(max_pos - 1, 0));
    const DiffRot rot{(cos_sin && rot_dims) ? cos_sin + (size_t)pos * rot_dims : nullptr, rot_dims, pairing};
    if (y < q_blocks) {
        TC* qo = q_out + (size_t)t * 2 * H * P;
        for (int hm = y * DQ_HEADS; hm < min(2 * H, (y + 1) * DQ_HEADS); ++hm) {
            const int lo = (hm & 1) * D;
            for (int e2 = tid; e2 < P; e2 += DQ_THREADS) {
                float v = 0.f;
                if (e2 >= lo && e2 < lo + D) v = diff_rotated(x + (size_t)hm * D, qb ? qb + (size_t)hm * D : nullptr, e2 - lo, rot);
                qo[(size_t)hm * P + e2] = from_f32<TC>(v);
            }
        }
        return;
    }
    const int slot = slots[t];
    if (slot < 0) return;      // (the whole block: a token that writes no key)
    const int g = y - q_blocks;
    const int page = slot / page_size, off = slot - page * page_size;
    const float* xk = x + (size_t)2 * H * D + (size_t)2 * g * D;
    const float* xv = x + (size_t)2 * H * D + (size_t)2 * G * D + (size_t)g * E;
    TC* kd = k_cache + (((size_t)page * G + g) * page_size + off) * P;
    TC* vd = v_cache + ((size_t)page * G + g) * P * page_size + off;
    for (int e2 = tid; e2 < P; e2 += DQ_THREADS) {
        float k = 0.f;
        if (e2 < 2 * D) {
            const int m = e2 >= D ? 1 : 0;
            k = diff_rotated(xk + (size_t)m * D, kb ? kb + (size_t)(2 * g + m) * D : nullptr, e2 - m * D, rot);
        }
        kd[e2] = from_f32<TC>(k);
        const float v = e2 < E ? xv[e2] + (vb ? vb[(size_t)g * E + e2] : 0.f) : 0.f;
        vd[(size_t)e2 * page_size] = from_f32<TC>(v);
    }
}

TFF_API int tff_diff_qkv_store(const float* proj, size_t row, const float* qb, const float* kb, const float* vb,
                               const float* cos_sin, int rot_dims, int pairing, int max_pos, const int32_t* positions,
                               const int32_t* slots, void* q_out, void* k_cache, void* v_cache, int page_size,
                               int num_pages, int T, int H, int G, int D, int E, int P, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(proj && positions && slots && q_out && k_cache && v_cache, "diff_qkv_store: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && E > 0, "diff_qkv_store: bad sizes H=%d G=%d D=%d E=%d", H, G, D, E);
    TFF_REQUIRE(P >= 2 * D && P >= E, "diff_qkv_store: a cache head of %d does not hold two maps of %d or values of %d", P, D, E);
    TFF_REQUIRE(row >= (size_t)2 * H * D + (size_t)2 * G * D + (size_t)G * E, "diff_qkv_store: rows of %zu are too short", row);
    TFF_REQUIRE(rot_dims >= 0 && rot_dims <= D && rot_dims % 2 == 0 && (rot_dims == 0 || (cos_sin && max_pos > 0)) &&
                (pairing == 0 || pairing == 1), "diff_qkv_store: %d rotated elements of a map of %d need an even count and a table", rot_dims, D);
    TFF_REQUIRE(page_size > 0 && num_pages > 0, "diff_qkv_store: bad cache geometry");
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int q_blocks = (2 * H + DQ_HEADS - 1) / DQ_HEADS;
    TFF_REQUIRE(q_blocks + G <= 65535, "diff_qkv_store: too many heads");
    const dim3 grid(T, q_blocks + G);
    if (dtype == TFF_F32)
        diff_qkv_store_kernel<float><<<grid, DQ_THREADS, 0, s>>>(proj, row, qb, kb, vb, cos_sin, rot_dims, pairing, max_pos, positions,
                                                                 slots, (float*)q_out, (float*)k_cache, (float*)v_cache, page_size,
                                                                 H, G, D, E, P, q_blocks);
    else if (dtype == TFF_BF16)
        diff_qkv_store_kernel<bf16_t><<<grid, DQ_THREADS, 0, s>>>(proj, row, qb, kb, vb, cos_sin, rot_dims, pairing, max_pos, positions,
                                                                  slots, (bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache,
                                                                  page_size, H, G, D, E, P, q_blocks);
    else
        return tff_fail("diff_qkv_store: unknown dtype %d", dtype);
    return tff_check_launch("diff_qkv_store");
}

// A wave per (token, head): o = a_0 - lambda a_1 over the head's E values, the sum of squares over the wave,
// out = o / sqrt(mean + eps) * out_scale * sigmoid(gate).
template <typename T>
__global__ __launch_bounds__(256) void diff_combine_kernel(const T* __restrict__ a, size_t a_row, int P,
                                                           const float* __restrict__ gate, size_t gate_row, float lambda,
                                                           float eps, float out_scale, T* __restrict__ out, size_t out_row,
                                                           int pairs, int H, int E) {
    const int lane = threadIdx.x & 63;
    const int pair = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (pair >= pairs) return;      // (a whole wave)
    const int t = pair / H, h = pair - t * H;
    const T* a0 = a + (size_t)t * a_row + (size_t)(2 * h) * P;
    const T* a1 = a0 + P;
    float ss = 0.f;
    for (int e = lane; e < E; e += 64) {
        const float o = fmaf(-lambda, to_f32(a1[e]), to_f32(a0[e]));
        ss = fmaf(o, o, ss);
    }
    ss = wave_sum(ss);
    const float f = out_scale / sqrtf(ss / (float)E + eps);
    for (int e = lane; e < E; e += 64) {
        float o = fmaf(-lambda, to_f32(a1[e]), to_f32(a0[e])) * f;
        if (gate) o *= 1.0f / (1.0f + expf(-gate[(size_t)t * gate_row + (size_t)h * E + e]));
        out[(size_t)t * out_row + (size_t)h * E + e] = from_f32<T>(o);
    }
}

TFF_API int tff_diff_combine(const void* a, size_t a_row, int P, const float* gate, size_t gate_row, float lambda, float eps,
                             float out_scale, void* out, size_t out_row, int T, int H, int E, int dtype, tff_stream_t stream) {
    TFF_REQUIRE(a && out, "diff_combine: null pointer");
    TFF_REQUIRE(T >= 0 && H > 0 && E > 0 && P >= E && a_row >= (size_t)2 * H * P && out_row >= (size_t)H * E &&
                (!gate || gate_row >= (size_t)H * E), "diff_combine: bad sizes H=%d E=%d P=%d", H, E, P);
    if (T == 0) return 0;
    hipStream_t s = (hipStream_t)stream;
    const int pairs = T * H;
    const unsigned blocks = (unsigned)((pairs + 3) / 4);
    if (dtype == TFF_F32)
        diff_combine_kernel<float><<<blocks, 256, 0, s>>>((const float*)a, a_row, P, gate, gate_row, lambda, eps, out_scale,
                                                          (float*)out, out_row, pairs, H, E);
    else if (dtype == TFF_BF16)
        diff_combine_kernel<bf16_t><<<blocks, 256, 0, s>>>((const bf16_t*)a, a_row, P, gate, gate_row, lambda, eps, out_scale,
                                                           (bf16_t*)out, out_row, pairs, H, E);
    else
        return tff_fail("diff_combine: unknown dtype %d", dtype);
    return tff_check_launch("diff_combine");
}
