// A feed-forward of many small experts of which every token uses a few ("mixture of experts").
//
// k_moe_route: per token, from the router's 32-bit logits (a matrix product of its own), a softmax over
// all experts, the `top` experts with the largest score + correction (ties: the lower index), and
// their weights: the chosen scores (without the correction) over their sum + 1e-20.  Options: the scores are
// sigmoid(logit), every expert for itself, instead of a softmax; the experts form `groups` equal groups of
// neighbours, a group's score is the sum of its two largest score + correction, and only experts of the `keep`
// groups that score highest can be chosen (ties: the lower group); the weights are the chosen scores times a
// given number instead of their share of their sum.
// k_moe_up / k_moe_down: the experts' two products token by token, a wave an output column, the
// weights of the chosen experts streamed: what a few decoded tokens need.  Expert:
// down(act(up h)), act = relu squared, or gated: down(silu(gate h) * (up h)) with the gate's rows before
// the up rows in one matrix [2F, E].  The down product adds a token's experts up in the order
// of its choice and writes (or adds to) 32-bit rows.
// k_moe_table_route: the choice without a router, a row of a table [vocab, top] by the token's id, every
// chosen expert with the same weight.
#include "common.h"

#define MOE_MAX_EXPERTS 1024
#define MOE_MAX_TOP 64      // lane j of the routing wave keeps the j-th choice

__global__ __launch_bounds__(64) void k_moe_route(int* __restrict__ idx, float* __restrict__ wts, const float* __restrict__ logits,
                                                  const float* __restrict__ correction, int ld, int n, int top, int sigmoid,
                                                  int groups, int keep, float weight_scale) {
    __shared__ float z[MOE_MAX_EXPERTS];
    __shared__ float gsc[MOE_MAX_EXPERTS];          // a group's score; then 1 if its experts can be chosen, else 0
    const int t = blockIdx.x, lane = threadIdx.x;
    for (int e = lane; e < n; e += 64) z[e] = logits[(size_t)t * ld + e];
    __syncthreads();
    if (sigmoid) {
        for (int e = lane; e < n; e += 64) z[e] = 1.0f / (1.0f + expf(-z[e]));      // the scores
    } else {
        float m = -INFINITY;
        for (int e = lane; e < n; e += 64) m = fmaxf(m, z[e]);
        m = wave_max(m);
        float l = 0.f;
        for (int e = lane; e < n; e += 64) l += expf(z[e] - m);
        l = wave_sum(l);
        __syncthreads();
        for (int e = lane; e < n; e += 64) z[e] = expf(z[e] - m) / l;       // the scores
    }
    __syncthreads();
    const int per = n / groups;
    if (groups > 1) {
        for (int g = lane; g < groups; g += 64) {
            float a = -INFINITY, b = -INFINITY;         // the group's two largest choice scores
            for (int e = g * per; e < (g + 1) * per; ++e) {
                float c = z[e] + correction[e];
                if (!(c == c)) c = -INFINITY;
                if (c > a) { b = a; a = c; } else if (c > b) b = c;
            }
            gsc[g] = per > 1 ? a + b : a;
        }
        __syncthreads();
        float mine_g[MOE_MAX_EXPERTS / 64];
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i) {
            const int g = lane + 64 * i;
            int rank = 0;
            if (g < groups)
                for (int o = 0; o < groups; ++o) rank += (gsc[o] > gsc[g] || (gsc[o] == gsc[g] && o < g)) ? 1 : 0;
            mine_g[i] = rank < keep ? 1.f : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < MOE_MAX_EXPERTS / 64; ++i)
            if (lane + 64 * i < groups) gsc[lane + 64 * i] = mine_g[i];
        __syncthreads();
    }
    // `top` passes of: the largest score + correction not yet taken, the lower index on a tie.  A score
    // that is no number (the row of a request that does not exist, whose state is whatever memory held)
    // counts as the smallest, so that every pass still finds an expert that exists.
    float total = 0.f;
    int mine = 0;           // lane j keeps the j-th choice
    float mine_s = 0.f;
    for (int j = 0; j < top; ++j) {
        float best = -INFINITY;
        int at = n;         // n: none found yet
        for (int e = lane; e < n; e += 64) {
            const float s = z[e];
            if (s < -0.5f) continue;        // taken: stored as -(s) - 1
            if (groups > 1 && gsc[e / per] == 0.f) continue;       // its group is out
            float c = s + correction[e];
            if (!(c == c)) c = -INFINITY;
            if (at == n || c > best || (c == best && e < at)) { best = c; at = e; }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (oa < n && (at == n || ob > best || (ob == best && oa < at))) { best = ob; at = oa; }
        }
        at = at < n ? at : 0;               // (top <= n: there is always one left; this is for the compiler and for memory that lies)
        float s = z[at];
        if (!(s == s) || s < 0.f) s = 0.f;
        total += s;
        if (lane == j) { mine = at; mine_s = s; }
        __syncthreads();
        if (lane == 0) z[at] = -s - 1.0f;
        __syncthreads();
    }
    if (lane < top) {
        idx[(size_t)t * top + lane] = mine;
        wts[(size_t)t * top + lane] = weight_scale > 0.f ? mine_s * weight_scale : mine_s / (total + 1e-20f);
    }
}

extern "C" int xr_moe_route(int* idx, float* wts, const float* logits, const float* correction, int T, int ld, int n, int top,
                            int sigmoid, int groups, int keep, float weight_scale, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && ld >= n, "moe_route: bad sizes T=%d ld=%d", T, ld);
    XR_REQUIRE(n >= 1 && n <= MOE_MAX_EXPERTS && top >= 1 && top <= n && top <= MOE_MAX_TOP,
               "moe_route: %d experts (at most %d), %d chosen (at most %d)", n, MOE_MAX_EXPERTS, top, MOE_MAX_TOP);
    XR_REQUIRE(groups >= 1 && n % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (n / groups),
               "moe_route: %d experts in %d groups of which %d are kept cannot give %d choices", n, groups, keep, top);
    XR_REQUIRE(weight_scale >= 0.f, "moe_route: weight scale %g (0: the chosen scores' shares of their sum)", (double)weight_scale);
    if (T == 0) return XR_OK;
    k_moe_route<<<T, 64, 0, stream>>>(idx, wts, logits, correction, ld, n, top, sigmoid, groups, keep, weight_scale);
    XR_CHECK_LAUNCH("moe_route");
    return XR_OK;
}

__global__ void k_moe_table_route(int* __restrict__ idx, float* __restrict__ wts, const int* __restrict__ table,
                                  const int* __restrict__ ids, int T, int V, int top, int n, float weight) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= T * top) return;
    const int t = i / top, j = i - t * top;
    int id = ids[t];
    id = id < 0 || id >= V ? 0 : id;                    // (as the embedding reads row 0 for an id outside the vocabulary)
    idx[i] = min(max(table[(size_t)id * top + j], 0), n - 1);
    wts[i] = weight;
}

extern "C" int xr_moe_table_route(int* idx, float* wts, const int* table, const int* ids, int T, int V, int top, int n,
                                  float weight, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && V > 0 && top >= 1 && n >= 1 && top <= MOE_MAX_TOP, "moe_table_route: bad sizes T=%d V=%d top=%d n=%d", T, V, top, n);
    XR_REQUIRE((long long)T * top <= 0x7fffffffLL, "moe_table_route: too many rows");
    if (T == 0) return XR_OK;
    k_moe_table_route<<<(T * top + 255) / 256, 256, 0, stream>>>(idx, wts, table, ids, T, V, top, n, weight);
    XR_CHECK_LAUNCH("moe_table_route");
    return XR_OK;
}

// A wave's dot product of two rows of n elements; `vec`: both rows start on 16 bytes and n is a multiple of
// 8 (bfloat16) or 4 (float), so a lane reads 16 bytes at a time.
template <typename TW> __device__ inline float wave_dot(const TW* __restrict__ w, const TW* __restrict__ x, int n, int lane, bool vec);
template <> __device__ inline float wave_dot<float>(const float* __restrict__ w, const float* __restrict__ x, int n, int lane, bool vec) {
    float acc = 0.f;
    if (vec) {
        for (int i = lane * 4; i < n; i += 256) {
            const float4 a = *reinterpret_cast<const float4*>(w + i), b = *reinterpret_cast<const float4*>(x + i);
            acc = fmaf(a.x, b.x, acc); acc = fmaf(a.y, b.y, acc); acc = fmaf(a.z, b.z, acc); acc = fmaf(a.w, b.w, acc);
        }
    } else {
        for (int i = lane; i < n; i += 64) acc = fmaf(w[i], x[i], acc);
    }
    return wave_sum(acc);
}
__device__ inline float bf_lo(uint32_t v) { return __uint_as_float(v << 16); }
__device__ inline float bf_hi(uint32_t v) { return __uint_as_float(v & 0xffff0000u); }
template <> __device__ inline float wave_dot<bf16_t>(const bf16_t* __restrict__ w, const bf16_t* __restrict__ x, int n, int lane, bool vec) {
    float acc = 0.f;
    if (vec) {
        for (int i = lane * 8; i < n; i += 512) {
            const uint4 a = *reinterpret_cast<const uint4*>(w + i), b = *reinterpret_cast<const uint4*>(x + i);
            acc = fmaf(bf_lo(a.x), bf_lo(b.x), acc); acc = fmaf(bf_hi(a.x), bf_hi(b.x), acc);
            acc = fmaf(bf_lo(a.y), bf_lo(b.y), acc); acc = fmaf(bf_hi(a.y), bf_hi(b.y), acc);
            acc = fmaf(bf_lo(a.z), bf_lo(b.z), acc); acc = fmaf(bf_hi(a.z), bf_hi(b.z), acc);
            acc = fmaf(bf_lo(a.w), bf_lo(b.w), acc); acc = fmaf(bf_hi(a.w), bf_hi(b.w), acc);
        }
    } else {
        for (int i = lane; i < n; i += 64) acc = fmaf(bf16_to_f32(w[i]), bf16_to_f32(x[i]), acc);
    }
    return wave_sum(acc);
}

// z[t * top + j][f] = relu(W_up[e][f] . h[t])^2 for e = idx[t][j]; `gated`: silu(W_up[e][f] . h[t]) * (W_up[e][F + f] . h[t]).
// Grid (T * top, ceil(F / 4)); a wave a column.
#define MOE_ACT_RELU2 0
#define MOE_ACT_SWIGLU 1
template <typename TW>
__global__ __launch_bounds__(256) void k_moe_up(TW* __restrict__ z, const TW* __restrict__ h, const TW* __restrict__ w_up,
                                                const int* __restrict__ idx, int E, int F, int ld_h, int top, int n, int vec,
                                                int gated) {
    const int a = blockIdx.x, f = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (f >= F) return;
    const int t = a / top, e = min(max(idx[a], 0), n - 1);
    const TW* row = h + (size_t)t * ld_h;
    const TW* w = w_up + ((size_t)e * (gated ? 2 * F : F) + f) * E;
    const float acc = wave_dot<TW>(w, row, E, lane, vec != 0);
    if (gated) {
        const float up = wave_dot<TW>(w + (size_t)F * E, row, E, lane, vec != 0);
        if (lane == 0) st<TW>(z, (size_t)a * F + f, gate_value<false>(XR_ACT_SILU, 0.f, acc, up));
        return;
    }
    if (lane == 0) {
        const float r = fmaxf(acc, 0.f);
        st<TW>(z, (size_t)a * F + f, r * r);
    }
}

// y[t][c] (+)= sum_j wts[t][j] * (W_down[e_j][c] . z[t * top + j]).  Grid (T, ceil(E / 4)); a wave a column.
template <typename TW>
__global__ __launch_bounds__(256) void k_moe_down(float* __restrict__ y, const TW* __restrict__ z, const TW* __restrict__ w_down,
                                                  const int* __restrict__ idx, const float* __restrict__ wts, int E, int F,
                                                  int ld_y, int top, int n, int accumulate, int vec) {
    const int t = blockIdx.x, c = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (c >= E) return;
    float sum = 0.f;
    for (int j = 0; j < top; ++j) {
        const int e = min(max(idx[(size_t)t * top + j], 0), n - 1);
        const TW* w = w_down + ((size_t)e * E + c) * F;
        const TW* zr = z + ((size_t)t * top + j) * F;
        sum += wts[(size_t)t * top + j] * wave_dot<TW>(w, zr, F, lane, vec != 0);
    }
    if (lane == 0) {
        float* o = y + (size_t)t * ld_y + c;
        *o = accumulate ? *o + sum : sum;
    }
}

extern "C" int xr_moe_experts(float* y, void* z, const void* h, const void* w_up, const void* w_down, const int* idx,
                              const float* wts, int T, int E, int F, int ld_h, int ld_y, int n, int top, int accumulate,
                              int dtype, int act, hipStream_t stream) {
    XR_REQUIRE(act == MOE_ACT_RELU2 || act == MOE_ACT_SWIGLU, "moe_experts: activation %d (0 = relu squared, 1 = SiLU-gated)", act);
    const int gated = act == MOE_ACT_SWIGLU;
    XR_REQUIRE(T >= 0 && E > 0 && F > 0 && ld_h >= E && ld_y >= E, "moe_experts: bad sizes T=%d E=%d F=%d", T, E, F);
    XR_REQUIRE(n >= 1 && top >= 1 && top <= n && top <= MOE_MAX_TOP, "moe_experts: %d experts, %d chosen", n, top);
    XR_REQUIRE((long long)T * top <= 0x7fffffffLL, "moe_experts: too many rows");
    if (T == 0) return XR_OK;
    const dim3 gu(T * top, (F + 3) / 4), gd(T, (E + 3) / 4);
    const int per16 = dtype == XR_BF16 ? 8 : 4;             // elements in 16 bytes
    const bool al = ((uintptr_t)h % 16) == 0 && ((uintptr_t)w_up % 16) == 0 && ((uintptr_t)w_down % 16) == 0 && ((uintptr_t)z % 16) == 0;
    const int vu = al && E % per16 == 0 && ld_h % per16 == 0, vd = al && F % per16 == 0;
    if (dtype == XR_F32) {
        k_moe_up<float><<<gu, 256, 0, stream>>>((float*)z, (const float*)h, (const float*)w_up, idx, E, F, ld_h, top, n, vu, gated);
        k_moe_down<float><<<gd, 256, 0, stream>>>(y, (const float*)z, (const float*)w_down, idx, wts, E, F, ld_y, top, n, accumulate, vd);
    } else if (dtype == XR_BF16) {
        k_moe_up<bf16_t><<<gu, 256, 0, stream>>>((bf16_t*)z, (const bf16_t*)h, (const bf16_t*)w_up, idx, E, F, ld_h, top, n, vu, gated);
        k_moe_down<bf16_t><<<gd, 256, 0, stream>>>(y, (const bf16_t*)z, (const bf16_t*)w_down, idx, wts, E, F, ld_y, top, n, accumulate, vd);
    } else { xr_set_error("moe_experts: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("moe_experts");
    return XR_OK;
}
