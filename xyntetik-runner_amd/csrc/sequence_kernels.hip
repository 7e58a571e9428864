// Row-wise and time-wise operations around the sequence mixers: layer norm, a short causal
// convolution over time with its carried inputs, the PolyNorm activation, a rotation of 32-bit
// projections in place, the gated norm of a recurrent mixer's read-out, and what a gated delta
// rule needs of its projections (unit vectors, write strengths, decays).
//
// All arithmetic is 32-bit; T is the storage type of what comes in or goes out.  A step's rows
// are the tokens of its requests one after another: request b owns rows cu_q[b] .. cu_q[b+1]-1
// and the state row slots[b].
#include "common.h"

// ---------------------------------------------------------------- layer norm
// y = (x - mean) / sqrt(var + eps) * w, var = mean((x - mean)^2); no bias.  One workgroup a row.
// NW waves a row: 4 where there are rows enough to fill the chip, 16 for the few rows of a
// decode step, whose time is the latency of one workgroup's passes over its row.
template <int NW> __device__ inline float block_sum(float v, float* part) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NW; ++i) t += part[i];
    return t;
}
#define FEW_ROWS 128

template <typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void k_layernorm(TO* __restrict__ out, const float* __restrict__ x,
                                                      const float* __restrict__ w, const int* __restrict__ rows,
                                                      int E, int ldx, float eps) {
    __shared__ float part[NW];
    const int r = blockIdx.x;
    const int src = rows ? rows[r] : r;
    const float* xr = x + (size_t)src * ldx;
    float s = 0.f;
    for (int i = threadIdx.x; i < E; i += 64 * NW) s += xr[i];
    const float mean = block_sum<NW>(s, part) / (float)E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 64 * NW) {
        const float d = xr[i] - mean;
        ss += d * d;
    }
    const float rinv = 1.0f / sqrtf(block_sum<NW>(ss, part) / (float)E + eps);
    TO* o = out + (size_t)r * E;
    for (int i = threadIdx.x; i < E; i += 64 * NW) st<TO>(o, i, (xr[i] - mean) * rinv * (w ? w[i] : 1.f));
}

extern "C" int xr_layernorm(void* out, const float* x, const float* w, const int* rows, int R, int E, int ldx,
                            float eps, int out_dtype, hipStream_t stream) {
    XR_REQUIRE(R >= 0 && E > 0 && ldx >= E, "layernorm: bad sizes R=%d E=%d ldx=%d", R, E, ldx);
    XR_REQUIRE(eps >= 0.f, "layernorm: eps %g is negative", eps);
    XR_REQUIRE(out_dtype == XR_F32 || out_dtype == XR_BF16, "layernorm: bad dtype %d", out_dtype);
    if (R == 0) return XR_OK;
    const bool few = R <= FEW_ROWS && E >= 1024;
    if (out_dtype == XR_F32) {
        if (few) k_layernorm<float, 16><<<R, 1024, 0, stream>>>((float*)out, x, w, rows, E, ldx, eps);
        else k_layernorm<float, 4><<<R, 256, 0, stream>>>((float*)out, x, w, rows, E, ldx, eps);
    } else {
        if (few) k_layernorm<bf16_t, 16><<<R, 1024, 0, stream>>>((bf16_t*)out, x, w, rows, E, ldx, eps);
        else k_layernorm<bf16_t, 4><<<R, 256, 0, stream>>>((bf16_t*)out, x, w, rows, E, ldx, eps);
    }
    XR_CHECK_LAUNCH("layernorm");
    return XR_OK;
}

// ---------------------------------------------------------------- short causal convolution over time
// y_t[c] = sum_j w[c][j] * u_(t - taps + 1 + j)[c]  (+ u_t[c] with `residual`), then the activation.
// Inputs before a portion's first row come from the request's state row, which holds its last
// taps - 1 inputs, oldest first, and is zero for a request that begins.  The state is rewritten by
// a second kernel once every row has been read; in a step where every request brings one row
// (`fuse`) a row's own thread is the only one that reads its request's state and rewrites it itself.
#define CONV_MAX_TAPS 16
#define XR_CONV_NONE 0
#define XR_CONV_SILU 1

template <typename TU, typename TO>
__global__ __launch_bounds__(256) void k_causal_conv(TO* __restrict__ out, const TU* __restrict__ u,
                                                     const float* __restrict__ w, TU* state,
                                                     const int* __restrict__ cu_q, const int* __restrict__ slots,
                                                     const int* __restrict__ req_of_token, int C, int taps, int ld_u,
                                                     int ld_out, int residual, int act, int fuse) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int b = req_of_token[t];
    const int row0 = cu_q[b];
    const int i = t - row0;
    TU* srow = state + (size_t)slots[b] * (taps - 1) * C;
    float acc = 0.f;
    for (int j = 0; j < taps; ++j) {
        const int s = i - (taps - 1) + j;
        const float val = s >= 0 ? ld<TU>(u, (size_t)(row0 + s) * ld_u + c) : ld<TU>(srow, (size_t)(taps - 1 + s) * C + c);
        acc = fmaf(w[(size_t)c * taps + j], val, acc);
        // one row a request: input j of this row is state entry j, which moves one place down
        if (fuse && j > 0) st<TU>(srow, (size_t)(j - 1) * C + c, val);
    }
    if (residual) acc += ld<TU>(u, (size_t)t * ld_u + c);
    if (act == XR_CONV_SILU) acc = acc / (1.0f + expf(-acc));
    st<TO>(out, (size_t)t * ld_out + c, acc);
}

// Many rows: a thread takes CONV_ROWS consecutive rows of its channel.  What a row needs before its
// first input (its request, the request's first row and state row) are three loads that wait for
// each other; with a row a thread a workgroup spent most of its life on them (2,048 rows of 2,048
// channels: 26 us), here the rows' chains run side by side.  (Four channels a thread with 16-byte
// loads was slower still: 34 us.)
#define CONV_ROWS 8
template <typename TU, typename TO>
__global__ __launch_bounds__(256) void k_causal_conv_rows(TO* __restrict__ out, const TU* __restrict__ u,
                                                          const float* __restrict__ w, const TU* __restrict__ state,
                                                          const int* __restrict__ cu_q, const int* __restrict__ slots,
                                                          const int* __restrict__ req_of_token, int T, int C, int taps,
                                                          int ld_u, int ld_out, int residual, int act) {
    const int t0 = blockIdx.y * CONV_ROWS;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    int row0[CONV_ROWS], slot[CONV_ROWS];
#pragma unroll
    for (int r = 0; r < CONV_ROWS; ++r) {
        const int b = req_of_token[t0 + r < T ? t0 + r : T - 1];
        row0[r] = cu_q[b];
        slot[r] = slots[b];
    }
    float wt[CONV_MAX_TAPS];
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) wt[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
#pragma unroll
    for (int r = 0; r < CONV_ROWS; ++r) {
        const int t = t0 + r;
        if (t >= T) break;
        const int i = t - row0[r];
        const TU* srow = state + (size_t)slot[r] * (taps - 1) * C;
        float acc = 0.f;
#pragma unroll
        for (int j = 0; j < CONV_MAX_TAPS; ++j) {
            if (j >= taps) break;
            const int s = i - (taps - 1) + j;
            const float val = s >= 0 ? ld<TU>(u, (size_t)(row0[r] + s) * ld_u + c) : ld<TU>(srow, (size_t)(taps - 1 + s) * C + c);
            acc = fmaf(wt[j], val, acc);
        }
        if (residual) acc += ld<TU>(u, (size_t)t * ld_u + c);
        if (act == XR_CONV_SILU) acc = acc / (1.0f + expf(-acc));
        st<TO>(out, (size_t)t * ld_out + c, acc);
    }
}

template <typename TU>
__global__ __launch_bounds__(256) void k_conv_state(TU* __restrict__ state, const TU* __restrict__ u,
                                                    const int* __restrict__ cu_q, const int* __restrict__ slots,
                                                    int C, int taps, int ld_u) {
    const int b = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    const int row0 = cu_q[b], n = cu_q[b + 1] - row0;
    if (n <= 0) return;
    TU* srow = state + (size_t)slots[b] * (taps - 1) * C;
    TU keep[CONV_MAX_TAPS];
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS; ++m) {
        if (m >= taps - 1) break;
        const int s = n - (taps - 1) + m;
        keep[m] = s >= 0 ? u[(size_t)(row0 + s) * ld_u + c] : srow[(size_t)(m + n) * C + c];
    }
#pragma unroll
    for (int m = 0; m < CONV_MAX_TAPS; ++m) {
        if (m >= taps - 1) break;
        srow[(size_t)m * C + c] = keep[m];
    }
}

extern "C" int xr_causal_conv(void* out, const void* u, const float* w, void* state, const int* cu_q, const int* slots,
                              const int* req_of_token, int T, int B, int C, int taps, int ld_u, int ld_out,
                              int u_dtype, int out_dtype, int residual, int act, int one_row_each, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && B >= 0 && C > 0 && ld_u >= C && ld_out >= C, "causal_conv: bad sizes T=%d B=%d C=%d ld_u=%d ld_out=%d",
               T, B, C, ld_u, ld_out);
    XR_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS, "causal_conv: %d taps (1 to %d)", taps, CONV_MAX_TAPS);
    XR_REQUIRE(act == XR_CONV_NONE || act == XR_CONV_SILU, "causal_conv: activation code %d", act);
    XR_REQUIRE(out != u, "causal_conv: the result cannot overwrite its input");
    XR_REQUIRE(taps == 1 || state != nullptr, "causal_conv: a convolution of %d taps needs its state", taps);
    XR_REQUIRE(!one_row_each || T == B, "causal_conv: %d rows of %d requests are not one row each", T, B);
    if (T == 0 || B == 0) return XR_OK;
    const int fuse = one_row_each && taps > 1 ? 1 : 0;
    dim3 grid((C + 255) / 256, T), sgrid((C + 255) / 256, B);
    dim3 rgrid((C + 255) / 256, (T + CONV_ROWS - 1) / CONV_ROWS);
#define CC(TU, TO)                                                                                                   \
    do {                                                                                                             \
        if (T >= 8 * CONV_ROWS && !fuse)                                                                             \
            k_causal_conv_rows<TU, TO><<<rgrid, 256, 0, stream>>>((TO*)out, (const TU*)u, w, (const TU*)state, cu_q,  \
                                                                  slots, req_of_token, T, C, taps, ld_u, ld_out,     \
                                                                  residual, act);                                    \
        else                                                                                                         \
        k_causal_conv<TU, TO><<<grid, 256, 0, stream>>>((TO*)out, (const TU*)u, w, (TU*)state, cu_q, slots,           \
                                                        req_of_token, C, taps, ld_u, ld_out, residual, act, fuse);    \
        if (taps > 1 && !fuse) k_conv_state<TU><<<sgrid, 256, 0, stream>>>((TU*)state, (const TU*)u, cu_q, slots, C, taps, ld_u); \
    } while (0)
    if (u_dtype == XR_F32 && out_dtype == XR_F32) CC(float, float);
    else if (u_dtype == XR_F32 && out_dtype == XR_BF16) CC(float, bf16_t);
    else if (u_dtype == XR_BF16 && out_dtype == XR_BF16) CC(bf16_t, bf16_t);
    else if (u_dtype == XR_BF16 && out_dtype == XR_F32) CC(bf16_t, float);
    else { xr_set_error("causal_conv: bad dtypes %d %d", u_dtype, out_dtype); return XR_BAD_ARG; }
#undef CC
    XR_CHECK_LAUNCH("causal_conv");
    return XR_OK;
}

// ---------------------------------------------------------------- mixes of a row with the row before it
// out[t][s][c] = h[t][c] + (h[t-1][c] - h[t][c]) * mu[s][c] for n mixes s ("token shift"); the row before a
// portion's first row is the request's state row (zero for a request that begins), which afterwards holds
// the portion's last row.  As for the convolution above, a second kernel rewrites the state once every row
// has been read, and in a step of one row a request (`fuse`) the row's own thread does.
template <typename TO>
__global__ __launch_bounds__(256) void k_token_shift(TO* __restrict__ out, const float* __restrict__ h,
                                                     const float* __restrict__ mu, float* state,
                                                     const int* __restrict__ cu_q, const int* __restrict__ slots,
                                                     const int* __restrict__ req_of_token, int E, int n, int ld_h, int fuse) {
    const int t = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= E) return;
    const int b = req_of_token[t];
    const bool first = t == cu_q[b];
    float* srow = state + (size_t)slots[b] * E;
    const float cur = h[(size_t)t * ld_h + c];
    const float before = first ? srow[c] : h[(size_t)(t - 1) * ld_h + c];
    const float d = before - cur;
    for (int s = 0; s < n; ++s) st<TO>(out, ((size_t)t * n + s) * E + c, fmaf(d, mu[(size_t)s * E + c], cur));
    if (fuse) srow[c] = cur;
}

__global__ __launch_bounds__(256) void k_shift_state(float* __restrict__ state, const float* __restrict__ h,
                                                     const int* __restrict__ cu_q, const int* __restrict__ slots, int E, int ld_h) {
    const int b = blockIdx.y;
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= E) return;
    const int end = cu_q[b + 1];
    if (end <= cu_q[b]) return;
    state[(size_t)slots[b] * E + c] = h[(size_t)(end - 1) * ld_h + c];
}

extern "C" int xr_token_shift(void* out, const float* h, const float* mu, float* state, const int* cu_q, const int* slots,
                              const int* req_of_token, int T, int B, int E, int n, int ld_h, int out_dtype, int one_row_each,
                              hipStream_t stream) {
    XR_REQUIRE(T >= 0 && B >= 0 && E > 0 && n > 0 && ld_h >= E, "token_shift: bad sizes T=%d B=%d E=%d n=%d ld=%d", T, B, E, n, ld_h);
    XR_REQUIRE(out && h && mu && state && cu_q && slots && req_of_token, "token_shift: a pointer is missing");
    XR_REQUIRE(!one_row_each || T == B, "token_shift: %d rows of %d requests are not one row each", T, B);
    XR_REQUIRE(out_dtype == XR_F32 || out_dtype == XR_BF16, "token_shift: bad dtype %d", out_dtype);
    if (T == 0 || B == 0) return XR_OK;
    const int fuse = one_row_each ? 1 : 0;
    const dim3 grid((E + 255) / 256, T), sgrid((E + 255) / 256, B);
    if (out_dtype == XR_F32) k_token_shift<float><<<grid, 256, 0, stream>>>((float*)out, h, mu, state, cu_q, slots, req_of_token, E, n, ld_h, fuse);
    else k_token_shift<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out, h, mu, state, cu_q, slots, req_of_token, E, n, ld_h, fuse);
    if (!fuse) k_shift_state<<<sgrid, 256, 0, stream>>>(state, h, cu_q, slots, E, ld_h);
    XR_CHECK_LAUNCH("token_shift");
    return XR_OK;
}

// Layer norm and the convolution behind it in one kernel, for a step in which every request
// brings one row: row b is request b's, its convolution reads the request's carried inputs and
// the row itself, and the thread that owns a channel moves that channel's carried inputs on.
//   h = layernorm(x);  y = h + sum_j cw[:, j] * (carried_j, ..., h);  carried <- (carried_1.., h)
template <typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void k_layernorm_conv(TO* __restrict__ out, const float* __restrict__ x,
                                                           const float* __restrict__ w, const float* __restrict__ cw,
                                                           float* state, const int* __restrict__ slots, int E, int ldx,
                                                           int taps, float eps) {
    __shared__ float part[NW];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)r * ldx;
    float s = 0.f;
    for (int i = threadIdx.x; i < E; i += 64 * NW) s += xr[i];
    const float mean = block_sum<NW>(s, part) / (float)E;
    float ss = 0.f;
    for (int i = threadIdx.x; i < E; i += 64 * NW) {
        const float d = xr[i] - mean;
        ss += d * d;
    }
    const float rinv = 1.0f / sqrtf(block_sum<NW>(ss, part) / (float)E + eps);
    float* srow = state + (size_t)slots[r] * (taps - 1) * E;
    TO* o = out + (size_t)r * E;
    for (int i = threadIdx.x; i < E; i += 64 * NW) {
        const float h = (xr[i] - mean) * rinv * (w ? w[i] : 1.f);
        float acc = 0.f;
        for (int j = 0; j < taps - 1; ++j) {
            const float val = srow[(size_t)j * E + i];
            acc = fmaf(cw[(size_t)i * taps + j], val, acc);
            if (j > 0) srow[(size_t)(j - 1) * E + i] = val;
        }
        acc = fmaf(cw[(size_t)i * taps + taps - 1], h, acc);
        if (taps > 1) srow[(size_t)(taps - 2) * E + i] = h;
        st<TO>(o, i, acc + h);
    }
}

extern "C" int xr_layernorm_conv(void* out, const float* x, const float* w, const float* cw, float* state,
                                 const int* slots, int R, int E, int ldx, int taps, float eps, int out_dtype,
                                 hipStream_t stream) {
    XR_REQUIRE(R >= 0 && E > 0 && ldx >= E, "layernorm_conv: bad sizes R=%d E=%d ldx=%d", R, E, ldx);
    XR_REQUIRE(taps >= 1 && taps <= CONV_MAX_TAPS && cw && slots && (taps == 1 || state), "layernorm_conv: %d taps, or an operand is missing", taps);
    XR_REQUIRE(out_dtype == XR_F32 || out_dtype == XR_BF16, "layernorm_conv: bad dtype %d", out_dtype);
    if (R == 0) return XR_OK;
    const bool few = R <= FEW_ROWS && E >= 1024;
    if (out_dtype == XR_F32) {
        if (few) k_layernorm_conv<float, 16><<<R, 1024, 0, stream>>>((float*)out, x, w, cw, state, slots, E, ldx, taps, eps);
        else k_layernorm_conv<float, 4><<<R, 256, 0, stream>>>((float*)out, x, w, cw, state, slots, E, ldx, taps, eps);
    } else {
        if (few) k_layernorm_conv<bf16_t, 16><<<R, 1024, 0, stream>>>((bf16_t*)out, x, w, cw, state, slots, E, ldx, taps, eps);
        else k_layernorm_conv<bf16_t, 4><<<R, 256, 0, stream>>>((bf16_t*)out, x, w, cw, state, slots, E, ldx, taps, eps);
    }
    XR_CHECK_LAUNCH("layernorm_conv");
    return XR_OK;
}

// ---------------------------------------------------------------- PolyNorm
// y = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N(v) = v / sqrt(mean(v^2) + eps)
// over the row.  One workgroup a row: the three sums in one pass, the result in a second.
template <typename TZ, typename TO, int NW>
__global__ __launch_bounds__(64 * NW) void k_polynorm(TO* __restrict__ out, const TZ* __restrict__ z,
                                                     const float* __restrict__ coef, int F, int ld_z, float eps) {
    __shared__ float part[NW];
    const TZ* zr = z + (size_t)blockIdx.x * ld_z;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    for (int i = threadIdx.x; i < F; i += 64 * NW) {
        const float v = ld<TZ>(zr, i), v2 = v * v, v3 = v2 * v;
        s2 += v2;
        s4 += v2 * v2;
        s6 += v3 * v3;
    }
    const float inv = 1.0f / (float)F;
    const float r1 = coef[0] / sqrtf(block_sum<NW>(s2, part) * inv + eps);
    const float r2 = coef[1] / sqrtf(block_sum<NW>(s4, part) * inv + eps);
    const float r3 = coef[2] / sqrtf(block_sum<NW>(s6, part) * inv + eps);
    const float e = coef[3];
    TO* o = out + (size_t)blockIdx.x * F;
    for (int i = threadIdx.x; i < F; i += 64 * NW) {
        const float v = ld<TZ>(zr, i), v2 = v * v;
        st<TO>(o, i, v * r1 + v2 * r2 + v2 * v * r3 + e);
    }
}

extern "C" int xr_polynorm(void* out, const void* z, const float* coef, int T, int F, int ld_z, float eps, int z_dtype,
                           int out_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && F > 0 && ld_z >= F, "polynorm: bad sizes T=%d F=%d ld=%d", T, F, ld_z);
    if (T == 0) return XR_OK;
    const bool few = T <= FEW_ROWS && F >= 1024;
#define PN(TZ, TO)                                                                                                        \
    do {                                                                                                                  \
        if (few) k_polynorm<TZ, TO, 16><<<T, 1024, 0, stream>>>((TO*)out, (const TZ*)z, coef, F, ld_z, eps);              \
        else k_polynorm<TZ, TO, 4><<<T, 256, 0, stream>>>((TO*)out, (const TZ*)z, coef, F, ld_z, eps);                    \
    } while (0)
    if (z_dtype == XR_F32 && out_dtype == XR_F32) PN(float, float);
    else if (z_dtype == XR_F32 && out_dtype == XR_BF16) PN(float, bf16_t);
    else if (z_dtype == XR_BF16 && out_dtype == XR_BF16) PN(bf16_t, bf16_t);
    else { xr_set_error("polynorm: bad dtypes %d %d", z_dtype, out_dtype); return XR_BAD_ARG; }
#undef PN
    XR_CHECK_LAUNCH("polynorm");
    return XR_OK;
}

// ---------------------------------------------------------------- rotation of 32-bit projections in place
// For every head of x [T, heads, D] (row stride ld): channel j < rot/2 pairs with j + rot/2,
// angle = position * inv_freq[j] as a 32-bit product; then every channel times `scale`.
__global__ __launch_bounds__(64) void k_rotate_rows(float* __restrict__ x, const int* __restrict__ positions,
                                                    const float* __restrict__ inv_freq, int D, int rot, int ld, float scale) {
    const int t = blockIdx.x, h = blockIdx.y;
    float* row = x + (size_t)t * ld + (size_t)h * D;
    const float pos = (float)positions[t];
    const int half = rot >> 1;
    for (int j = threadIdx.x; j < half; j += 64) {
        const float a = pos * inv_freq[j];
        const float c = cosf(a), s = sinf(a);
        const float u = row[j], v = row[j + half];
        row[j] = (u * c - v * s) * scale;
        row[j + half] = (v * c + u * s) * scale;
    }
    if (scale != 1.0f)
        for (int d = rot + threadIdx.x; d < D; d += 64) row[d] *= scale;
}

extern "C" int xr_rotate_rows(float* x, const int* positions, const float* inv_freq, int T, int heads, int D, int rot,
                              int ld, float scale, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && heads > 0 && D > 0 && ld >= heads * D, "rotate_rows: bad sizes T=%d heads=%d D=%d ld=%d", T, heads, D, ld);
    XR_REQUIRE(rot >= 0 && rot <= D && rot % 2 == 0, "rotate_rows: rotary width %d does not fit head size %d", rot, D);
    XR_REQUIRE(rot == 0 || inv_freq != nullptr, "rotate_rows: no frequency table");
    if (T == 0 || (rot == 0 && scale == 1.0f)) return XR_OK;
    k_rotate_rows<<<dim3(T, heads), 64, 0, stream>>>(x, positions, inv_freq, D, rot, ld, scale);
    XR_CHECK_LAUNCH("rotate_rows");
    return XR_OK;
}

// ---------------------------------------------------------------- gated norm of a read-out
// out[t][h][d] = o[t][h][d] / sqrt(mean_d(o^2) + eps) * w * act(gate[t][h][d]); w may be absent, is one
// weight a channel of a head that the heads share (w [Dv]) or, with w_full, one a channel of the row
// (w [H * Dv]); act is SiLU (gate_act 0) or the sigmoid (1).  A norm over all heads together is
// H = 1 with Dv the whole row.  One wave per (token, head).
#define XR_GATE_SILU 0
#define XR_GATE_SIGMOID 1
template <typename TO>
__global__ __launch_bounds__(64) void k_gated_rmsnorm(TO* __restrict__ out, const float* __restrict__ o,
                                                      const float* __restrict__ gate, const float* __restrict__ w,
                                                      int H, int Dv, int ld_g, float eps, int w_full, int gate_act) {
    const int t = blockIdx.x, h = blockIdx.y;
    const float* orow = o + ((size_t)t * H + h) * Dv;
    const float* grow = gate + (size_t)t * ld_g + (size_t)h * Dv;
    const float* wrow = w ? (w_full ? w + (size_t)h * Dv : w) : nullptr;
    float ss = 0.f;
    for (int d = threadIdx.x; d < Dv; d += 64) ss += orow[d] * orow[d];
    const float rinv = 1.0f / sqrtf(wave_sum(ss) / (float)Dv + eps);
    TO* dst = out + ((size_t)t * H + h) * Dv;
    for (int d = threadIdx.x; d < Dv; d += 64) {
        const float g = grow[d];
        const float sg = 1.0f / (1.0f + expf(-g));
        st<TO>(dst, d, orow[d] * rinv * (wrow ? wrow[d] : 1.f) * (gate_act == XR_GATE_SIGMOID ? sg : g * sg));
    }
}

// The same with a workgroup of 256 a (token, head), for long rows (all heads normed together).
template <typename TO>
__global__ __launch_bounds__(256) void k_gated_rmsnorm_wide(TO* __restrict__ out, const float* __restrict__ o,
                                                           const float* __restrict__ gate, const float* __restrict__ w,
                                                           int H, int Dv, int ld_g, float eps, int w_full, int gate_act) {
    __shared__ float part[4];
    const int t = blockIdx.x, h = blockIdx.y;
    const float* orow = o + ((size_t)t * H + h) * Dv;
    const float* grow = gate + (size_t)t * ld_g + (size_t)h * Dv;
    const float* wrow = w ? (w_full ? w + (size_t)h * Dv : w) : nullptr;
    float ss = 0.f;
    for (int d = threadIdx.x; d < Dv; d += 256) ss += orow[d] * orow[d];
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
    __syncthreads();
    const float rinv = 1.0f / sqrtf(((part[0] + part[1]) + (part[2] + part[3])) / (float)Dv + eps);
    TO* dst = out + ((size_t)t * H + h) * Dv;
    for (int d = threadIdx.x; d < Dv; d += 256) {
        const float g = grow[d];
        const float sg = 1.0f / (1.0f + expf(-g));
        st<TO>(dst, d, orow[d] * rinv * (wrow ? wrow[d] : 1.f) * (gate_act == XR_GATE_SIGMOID ? sg : g * sg));
    }
}

extern "C" int xr_gated_rmsnorm(void* out, const float* o, const float* gate, const float* w, int T, int H, int Dv,
                                int ld_g, float eps, int out_dtype, int w_full, int gate_act, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && Dv > 0 && ld_g >= H * Dv, "gated_rmsnorm: bad sizes T=%d H=%d Dv=%d ld=%d", T, H, Dv, ld_g);
    XR_REQUIRE(gate_act == XR_GATE_SILU || gate_act == XR_GATE_SIGMOID, "gated_rmsnorm: unknown gate activation %d", gate_act);
    if (T == 0) return XR_OK;
    const bool wide = Dv > 256;       // (the sums' order differs between the two kernels, not between calls of one size)
    if (out_dtype == XR_F32 && wide) k_gated_rmsnorm_wide<float><<<dim3(T, H), 256, 0, stream>>>((float*)out, o, gate, w, H, Dv, ld_g, eps, w_full, gate_act);
    else if (out_dtype == XR_BF16 && wide) k_gated_rmsnorm_wide<bf16_t><<<dim3(T, H), 256, 0, stream>>>((bf16_t*)out, o, gate, w, H, Dv, ld_g, eps, w_full, gate_act);
    else if (out_dtype == XR_F32) k_gated_rmsnorm<float><<<dim3(T, H), 64, 0, stream>>>((float*)out, o, gate, w, H, Dv, ld_g, eps, w_full, gate_act);
    else if (out_dtype == XR_BF16) k_gated_rmsnorm<bf16_t><<<dim3(T, H), 64, 0, stream>>>((bf16_t*)out, o, gate, w, H, Dv, ld_g, eps, w_full, gate_act);
    else { xr_set_error("gated_rmsnorm: bad dtype %d", out_dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("gated_rmsnorm");
    return XR_OK;
}

// ---------------------------------------------------------------- an activation on 32-bit rows
// x[t][c] <- act(x[t][c]) for the first W columns of rows of stride ld, in place; or, with `out`, into
// contiguous rows [T, W] of the type the next product reads.  act 1 = SiLU, 2 = tanh.
#define XR_ACT_ROWS_TANH 2
template <typename TO>
__global__ void k_act_rows(float* __restrict__ x, TO* __restrict__ out, int W, int ld, size_t n, int act) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / W;
    float* p = x + t * ld + (i - t * W);
    const float v = *p;
    const float y = act == XR_ACT_ROWS_TANH ? tanhf(v) : v / (1.0f + expf(-v));
    if (out) st<TO>(out, i, y);
    else *p = y;
}

extern "C" int xr_act_rows(float* x, int T, int W, int ld, int act, void* out, int out_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && W > 0 && ld >= W, "act_rows: bad sizes T=%d W=%d ld=%d", T, W, ld);
    XR_REQUIRE(act == XR_CONV_SILU || act == XR_ACT_ROWS_TANH, "act_rows: activation %d is not built (1 = SiLU, 2 = tanh)", act);
    XR_REQUIRE(!out || out_dtype == XR_F32 || out_dtype == XR_BF16, "act_rows: output type %d", out_dtype);
    const size_t n = (size_t)T * W;
    if (n == 0) return XR_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (out && out_dtype == XR_BF16) k_act_rows<bf16_t><<<blocks, 256, 0, stream>>>(x, (bf16_t*)out, W, ld, n, act);
    else k_act_rows<float><<<blocks, 256, 0, stream>>>(x, (float*)out, W, ld, n, act);
    XR_CHECK_LAUNCH("act_rows");
    return XR_OK;
}

// ---------------------------------------------------------------- what a gated delta rule reads
// In place on 32-bit rows (queries and keys of row stride ld, b and a of row stride ld_g): every query and key head becomes a unit vector
// x / sqrt(sum(x^2) + unit_eps), queries also times q_scale; the write strength of head h becomes
// sigmoid(b), its decay exp(-exp(a_log[h]) * softplus(a + dt_bias[h])).
__global__ __launch_bounds__(64) void k_delta_prepare(float* __restrict__ q, float* __restrict__ k, float* __restrict__ b,
                                                      float* __restrict__ a, const float* __restrict__ a_log,
                                                      const float* __restrict__ dt_bias, int G, int H, int D, int ld,
                                                      int ld_g, float q_scale, float unit_eps) {
    const int t = blockIdx.x, y = blockIdx.y;
    if (y < 2 * G) {
        float* row = (y < G ? q : k) + (size_t)t * ld + (size_t)(y < G ? y : y - G) * D;
        float ss = 0.f;
        for (int d = threadIdx.x; d < D; d += 64) ss += row[d] * row[d];
        const float f = (y < G ? q_scale : 1.0f) / sqrtf(wave_sum(ss) + unit_eps);
        for (int d = threadIdx.x; d < D; d += 64) row[d] *= f;
        return;
    }
    for (int h = threadIdx.x; h < H; h += 64) {
        const size_t i = (size_t)t * ld_g + h;
        b[i] = 1.0f / (1.0f + expf(-b[i]));
        if (!a) continue;           // (the decays are made elsewhere: one a key channel, say)
        const float z = a[i] + dt_bias[h];
        const float sp = z > 20.0f ? z : log1pf(expf(z));
        a[i] = expf(-expf(a_log[h]) * sp);
    }
}

extern "C" int xr_delta_prepare(float* q, float* k, float* b, float* a, const float* a_log, const float* dt_bias, int T,
                                int G, int H, int D, int ld, int ld_g, float q_scale, float unit_eps, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && G > 0 && H > 0 && D > 0 && ld >= G * D && ld_g >= H, "delta_prepare: bad sizes T=%d G=%d H=%d D=%d ld=%d ld_g=%d",
               T, G, H, D, ld, ld_g);
    if (T == 0) return XR_OK;
    k_delta_prepare<<<dim3(T, 2 * G + 1), 64, 0, stream>>>(q, k, b, a, a_log, dt_bias, G, H, D, ld, ld_g, q_scale, unit_eps);
    XR_CHECK_LAUNCH("delta_prepare");
    return XR_OK;
}
