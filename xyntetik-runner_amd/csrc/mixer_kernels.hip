// Small kernels around mixers that run side by side and around attention with a sink, a gate a head or
// tokens that a window keeps; all arithmetic in 32 bits.
//
// k_decay_prepare:   the decays of a recurrence whose decay is a number a token, head and key channel, made in
//                    place from the 32-bit rows of their projection:
//                      form 0: sigmoid(z)^(1/tau) = exp(-softplus(-z) / tau)
//                      form 1: exp(-exp(A_log[h]) * softplus(z + dt_bias[h, c]))
// k_head_gate:       an attention's output times sigmoid(g) with one g a token and head, in place.
// k_pair_combine:    x += a_l f(y_l) + a_r f(y_r) for two mixers' 32-bit results, f the identity or an RMS norm over
//                    the row with a weight of its own a side; and, if asked, the RMS norm of the updated row times
//                    a weight (the norm that the next sublayer reads through) in the same pass.
// k_add_rows:        x[t] += s y[t] + v, a vector added to every row (y absent: the vector alone).
// k_attn_extra_partial: for the matrix-core attention kernels, which take a window's (or a chunk's) keys: what else
//                    enters the same softmax, as a partial result of its own that their merge adds: a sink (a score
//                    without key or value, one a head) and the first `keep` keys of the request where the
//                    window has passed them.
#include "common.h"

#define MK_MAX_D 256

__device__ inline float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

__global__ void k_decay_prepare(float* __restrict__ x, int W, int ld, size_t n, int form, float inv_tau,
                                const float* __restrict__ a_log, const float* __restrict__ dt_bias, int D) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / W;
    const int c = (int)(i - t * W);
    float* p = x + t * ld + c;
    const float z = *p;
    if (form == 0) *p = expf(-softplus_f(-z) * inv_tau);
    else *p = expf(-expf(a_log[c / D]) * softplus_f(z + dt_bias[c]));
}

extern "C" int xr_decay_prepare(float* x, int T, int H, int D, int ld, int form, float tau, const float* a_log,
                                const float* dt_bias, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && D > 0 && ld >= H * D, "decay_prepare: bad sizes T=%d H=%d D=%d ld=%d", T, H, D, ld);
    XR_REQUIRE(form == 0 || form == 1, "decay_prepare: form %d (0: sigmoid to the power 1/tau, 1: exp(-exp(A) softplus))", form);
    XR_REQUIRE(form != 0 || tau > 0.f, "decay_prepare: tau %g must be positive", tau);
    XR_REQUIRE(form != 1 || (a_log && dt_bias), "decay_prepare: form 1 needs A_log and dt_bias");
    const size_t n = (size_t)T * H * D;
    if (n == 0) return XR_OK;
    k_decay_prepare<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, H * D, ld, n, form, form == 0 ? 1.0f / tau : 0.f, a_log, dt_bias, D);
    XR_CHECK_LAUNCH("decay_prepare");
    return XR_OK;
}

template <typename T>
__global__ void k_head_gate(T* __restrict__ o, const float* __restrict__ g, int H, int Dv, int ld_g, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t th = i / Dv;               // token * H + head
    const size_t t = th / H;
    const float z = g[t * ld_g + (th - t * H)];
    st<T>(o, i, ld<T>(o, i) / (1.0f + expf(-z)));
}

extern "C" int xr_head_gate(void* o, const float* g, int T, int H, int Dv, int ld_g, int dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && Dv > 0 && ld_g >= H, "head_gate: bad sizes T=%d H=%d Dv=%d ld=%d", T, H, Dv, ld_g);
    const size_t n = (size_t)T * H * Dv;
    if (n == 0) return XR_OK;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == XR_F32) k_head_gate<float><<<blocks, 256, 0, stream>>>((float*)o, g, H, Dv, ld_g, n);
    else if (dtype == XR_BF16) k_head_gate<bf16_t><<<blocks, 256, 0, stream>>>((bf16_t*)o, g, H, Dv, ld_g, n);
    else { xr_set_error("head_gate: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("head_gate");
    return XR_OK;
}

// One workgroup a row.  With `normed` each side is first divided by its root mean square over the row (eps
// inside the root) and multiplied by its weight.  With `h` the updated row over its root mean square (eps_h inside
// the root) times w_h goes there as well.
template <typename TO>
__global__ __launch_bounds__(256) void k_pair_combine(float* __restrict__ x, const float* __restrict__ yl,
                                                      const float* __restrict__ yr, const float* __restrict__ wl,
                                                      const float* __restrict__ wr, float al, float ar, float eps, int E,
                                                      int ld_x, int normed, TO* __restrict__ h,
                                                      const float* __restrict__ w_h, float eps_h) {
    __shared__ float part[3][4];
    const int t = blockIdx.x;
    const float* l = yl + (size_t)t * E;
    const float* r = yr + (size_t)t * E;
    float fl = al, fr = ar;
    if (normed) {
        float sl = 0.f, sr = 0.f;
        for (int c = threadIdx.x; c < E; c += 256) { sl = fmaf(l[c], l[c], sl); sr = fmaf(r[c], r[c], sr); }
        sl = wave_sum(sl); sr = wave_sum(sr);
        if ((threadIdx.x & 63) == 0) { part[0][threadIdx.x >> 6] = sl; part[1][threadIdx.x >> 6] = sr; }
        __syncthreads();
        fl *= 1.0f / sqrtf(((part[0][0] + part[0][1]) + (part[0][2] + part[0][3])) / (float)E + eps);
        fr *= 1.0f / sqrtf(((part[1][0] + part[1][1]) + (part[1][2] + part[1][3])) / (float)E + eps);
    }
    float* xr = x + (size_t)t * ld_x;
    float sx = 0.f;
    for (int c = threadIdx.x; c < E; c += 256) {
        const float a = l[c] * fl * (normed ? wl[c] : 1.f), b = r[c] * fr * (normed ? wr[c] : 1.f);
        const float v = xr[c] + (a + b);
        xr[c] = v;
        sx = fmaf(v, v, sx);
    }
    if (!h) return;
    sx = wave_sum(sx);
    if ((threadIdx.x & 63) == 0) part[2][threadIdx.x >> 6] = sx;
    __syncthreads();
    const float fh = 1.0f / sqrtf(((part[2][0] + part[2][1]) + (part[2][2] + part[2][3])) / (float)E + eps_h);
    for (int c = threadIdx.x; c < E; c += 256) st<TO>(h, (size_t)t * E + c, xr[c] * fh * w_h[c]);      // (each thread reads what it wrote)
}

extern "C" int xr_pair_combine(float* x, const float* yl, const float* yr, const float* wl, const float* wr, float al,
                               float ar, float eps, int T, int E, int ld_x, int normed, void* h, const float* w_h,
                               float eps_h, int h_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && ld_x >= E && x && yl && yr, "pair_combine: bad sizes T=%d E=%d ld=%d", T, E, ld_x);
    XR_REQUIRE(!normed || (wl && wr), "pair_combine: a norm a side needs its weight");
    XR_REQUIRE(!h || (w_h && (h_dtype == XR_F32 || h_dtype == XR_BF16)), "pair_combine: the norm of the sum needs a weight and an output type");
    if (T == 0) return XR_OK;
    if (h && h_dtype == XR_BF16)
        k_pair_combine<bf16_t><<<T, 256, 0, stream>>>(x, yl, yr, wl, wr, al, ar, eps, E, ld_x, normed, (bf16_t*)h, w_h, eps_h);
    else
        k_pair_combine<float><<<T, 256, 0, stream>>>(x, yl, yr, wl, wr, al, ar, eps, E, ld_x, normed, (float*)h, w_h, eps_h);
    XR_CHECK_LAUNCH("pair_combine");
    return XR_OK;
}

__global__ void k_add_rows(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ v, float s, int E,
                           size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float a = x[i] + v[i % E];
    if (y) a = fmaf(s, y[i], a);
    x[i] = a;
}

extern "C" int xr_add_rows(float* x, const float* y, const float* v, float s, int T, int E, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && x && v, "add_rows: bad sizes T=%d E=%d", T, E);
    const size_t n = (size_t)T * E;
    if (n == 0) return XR_OK;
    k_add_rows<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(x, y, v, s, E, n);
    XR_CHECK_LAUNCH("add_rows");
    return XR_OK;
}

// A record of `extras` names a block of 32 rows (row = token x heads-in-group + head) and its slot: request, row0,
// slot, q0, q_len, start.  One wave a row: the scores of the kept keys below the row's own range, a lane a key,
// then the sink; the result lies where the matrix-core kernels leave a key range's (part_o [slot][kv_head][32][D]
// the normalised output, part_ml the reference in units of log2 and the sum).  A row with neither leaves an empty
// partial result (sum 0), which the merge passes over.
struct ExtraArgs {
    const int* block_table;
    int table_stride, H, Hk, D, page_shift, page_mask, page_size;
    float scale;
    int window, chunk, keep;
    const float* sinks;     // [H] or null
    const float* slopes;    // [H] or null
};

__device__ inline int mask_lo(int pos, int window, int chunk) {
    if (chunk > 0) return pos - pos % chunk;
    return (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
}

template <typename T>
__global__ __launch_bounds__(256) void k_attn_extra_partial(float* __restrict__ part_o, float* __restrict__ part_ml,
                                                            const T* __restrict__ q, const T* __restrict__ kc,
                                                            const T* __restrict__ vc, const int* __restrict__ extras,
                                                            ExtraArgs a) {
    __shared__ float qs[4][MK_MAX_D];
    const int* ex = extras + (size_t)(blockIdx.x >> 3) * 8;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = (blockIdx.x & 7) * 4 + wave;
    const int kvh = blockIdx.y, G = a.H / a.Hk;
    const int req = ex[0], rho = ex[1] + r, slot = ex[2], q0 = ex[3], q_len = ex[4], start = ex[5];
    const int tok = rho / G, hg = rho - tok * G;
    const bool row = tok < q_len;
    const int h = kvh * G + hg;
    if (row) {
        const T* qrow = q + ((size_t)(q0 + tok) * a.H + h) * a.D;
        for (int d = lane; d < a.D; d += 64) qs[wave][d] = ld<T>(qrow, d);
    }
    __syncthreads();
    if (!row) return;
    const int pos = start + tok;
    const int lo = mask_lo(pos, a.window, a.chunk);
    const int hi = a.keep < lo ? a.keep : lo;           // kept keys [0, hi) lie below the row's own range
    const int* bt = a.block_table + (size_t)req * a.table_stride;
    const float slope = a.slopes ? a.slopes[h] : 0.f;
    float m = a.sinks ? a.sinks[h] : -INFINITY, l = a.sinks ? 1.f : 0.f;
    float acc[MK_MAX_D / 64];
#pragma unroll
    for (int dd = 0; dd < MK_MAX_D / 64; ++dd) acc[dd] = 0.f;
    // A few kept keys (the usual case): key by key, the lanes sharing a key's channels, so that the whole wave works;
    // many: a lane a key, as the 32-bit attention kernel does.  Which of the two runs depends on the row's position alone.
    for (int j = 0; hi <= 16 && j < hi; ++j) {
        const int page = bt[j >> a.page_shift], off = j & a.page_mask;
        const T* kr = kc + (((size_t)page * a.Hk + kvh) * a.page_size + off) * a.D;
        float dot = 0.f;
        for (int d = lane; d < a.D; d += 64) dot = fmaf(qs[wave][d], ld<T>(kr, d), dot);
        const float s = wave_sum(dot) * a.scale - slope * (float)(pos - j);
        const float mn = fmaxf(m, s);
        const float p = expf(s - mn);
        const float corr = m == -INFINITY ? 0.f : expf(m - mn);
        l = l * corr + p;
        const T* vb = vc + ((size_t)page * a.Hk + kvh) * a.D * a.page_size + off;
#pragma unroll
        for (int dd = 0; dd < MK_MAX_D / 64; ++dd) {
            const int d = lane + 64 * dd;
            if (d < a.D) acc[dd] = fmaf(p, ld<T>(vb, (size_t)d * a.page_size), acc[dd] * corr);
        }
        m = mn;
    }
    for (int k0 = hi <= 16 ? hi : 0; k0 < hi; k0 += 64) {
        const int key = k0 + lane;
        const bool valid = key < hi;
        float s = -INFINITY;
        if (valid) {
            const T* kr = kc + (((size_t)bt[key >> a.page_shift] * a.Hk + kvh) * a.page_size + (key & a.page_mask)) * a.D;
            float dot = 0.f;
            for (int d = 0; d < a.D; ++d) dot = fmaf(qs[wave][d], ld<T>(kr, d), dot);
            s = dot * a.scale - slope * (float)(pos - key);
        }
        const float mn = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - mn) : 0.f;
        const float corr = m == -INFINITY ? 0.f : expf(m - mn);
        l = l * corr + wave_sum(p);
#pragma unroll
        for (int dd = 0; dd < MK_MAX_D / 64; ++dd) acc[dd] *= corr;
        const int nk = hi - k0 < 64 ? hi - k0 : 64;
        for (int j = 0; j < nk; ++j) {
            const float pj = __shfl(p, j, 64);
            const int kj = k0 + j;
            const T* vb = vc + ((size_t)bt[kj >> a.page_shift] * a.Hk + kvh) * a.D * a.page_size + (kj & a.page_mask);
#pragma unroll
            for (int dd = 0; dd < MK_MAX_D / 64; ++dd) {
                const int d = lane + 64 * dd;
                if (d < a.D) acc[dd] = fmaf(pj, ld<T>(vb, (size_t)d * a.page_size), acc[dd]);
            }
        }
        m = mn;
    }
    const size_t at = ((size_t)slot * a.Hk + kvh) * 32 + r;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int dd = 0; dd < MK_MAX_D / 64; ++dd) {
        const int d = lane + 64 * dd;
        if (d < a.D) part_o[at * a.D + d] = acc[dd] * inv;
    }
    if (lane == 0) {
        part_ml[at * 2] = m * 1.44269504f;
        part_ml[at * 2 + 1] = l;
    }
}

extern "C" int xr_attn_extra_partial(float* part_o, float* part_ml, const void* q, const void* k_cache, const void* v_cache,
                                     const int* extras, int n_extras, const int* block_table, int table_stride, int H,
                                     int Hk, int D, int page_size, float scale, int window, int chunk, int keep,
                                     const float* sinks, const float* slopes, int dtype, hipStream_t stream) {
    XR_REQUIRE(n_extras >= 0 && H > 0 && Hk > 0 && H % Hk == 0, "attention extras: %d query heads over %d key/value heads", H, Hk);
    XR_REQUIRE(D > 0 && D <= MK_MAX_D, "attention extras: head size %d (1 to %d)", D, MK_MAX_D);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "attention extras: page size %d is not a power of two", page_size);
    XR_REQUIRE(window >= 0 && chunk >= 0 && keep >= 0, "attention extras: window %d, chunk %d, kept %d", window, chunk, keep);
    XR_REQUIRE(part_o && part_ml && q && extras && (keep == 0 || (k_cache && v_cache && block_table)), "attention extras: an operand is missing");
    if (n_extras == 0) return XR_OK;
    ExtraArgs a{block_table, table_stride, H, Hk, D, shift, page_size - 1, page_size, scale, window, chunk, keep, sinks, slopes};
    dim3 grid((unsigned)n_extras * 8, Hk);
    if (dtype == XR_F32)
        k_attn_extra_partial<float><<<grid, 256, 0, stream>>>(part_o, part_ml, (const float*)q, (const float*)k_cache, (const float*)v_cache, extras, a);
    else if (dtype == XR_BF16)
        k_attn_extra_partial<bf16_t><<<grid, 256, 0, stream>>>(part_o, part_ml, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, extras, a);
    else { xr_set_error("attention extras: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("attn_extra_partial");
    return XR_OK;
}
