// Sliding-window attention with pooled blocks over the paged cache, 32-bit arithmetic.
//
// The query at position p of its request attends to two kinds of entries in a single softmax:
// the cached keys at positions j, p - size < j <= p, and one summary per block of P positions
// whose last position b P + P - 1 is at most p - size: the arithmetic means of that block's cached
// keys and of its cached values.  Positions older than the window whose block is still
// incomplete, or not yet far enough back, contribute nothing.  P = 0: no summaries.
//
// The means live in a cache of their own with one entry a block (entry b of a request at place
// b of its own block table); k_pool_blocks writes the entries of the blocks a step completes,
// from the cache pages, once the step's keys and values are stored.  Key size D and value size
// Dv may differ.  Cache layout: K [page][kv_head][slot][D], V [page][kv_head][Dv][slot].
#include "common.h"

#define AP_MAX_D 512

// ---------------------------------------------------------------- queries out, keys and values into their pages
template <typename T>
__global__ __launch_bounds__(256) void k_qkv_store(T* __restrict__ q_out, T* __restrict__ kc, T* __restrict__ vc,
                                                   const float* __restrict__ q, const float* __restrict__ k,
                                                   const float* __restrict__ v, int ld, const int* __restrict__ positions,
                                                   const int* __restrict__ req_of_token, const int* __restrict__ block_table,
                                                   int table_stride, int Q, int Hk, int D, int Dv, int page_shift,
                                                   int page_mask, int page_size) {
    const int t = blockIdx.x;
    const float* qr = q + (size_t)t * ld;
    for (int i = threadIdx.x; i < Q; i += 256) st<T>(q_out, (size_t)t * Q + i, qr[i]);
    if (Hk == 0) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)req_of_token[t] * table_stride + (pos >> page_shift)];
    const int off = pos & page_mask;
    const float* kr = k + (size_t)t * ld;
    const float* vr = v + (size_t)t * ld;
    for (int i = threadIdx.x; i < Hk * D; i += 256) {
        const int h = i / D, d = i - h * D;
        st<T>(kc, (((size_t)page * Hk + h) * page_size + off) * D + d, kr[i]);
    }
    for (int i = threadIdx.x; i < Hk * Dv; i += 256) {
        const int h = i / Dv, d = i - h * Dv;
        st<T>(vc, (((size_t)page * Hk + h) * Dv + d) * page_size + off, vr[i]);
    }
}

extern "C" int xr_qkv_store(void* q_out, void* k_cache, void* v_cache, const float* q, const float* k, const float* v,
                            int ld, const int* positions, const int* req_of_token, const int* block_table,
                            int table_stride, int T, int H, int Hk, int D, int Dv, int page_size, int dtype,
                            hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && Hk >= 0 && D > 0 && Dv > 0, "qkv_store: bad sizes T=%d H=%d Hk=%d D=%d Dv=%d", T, H, Hk, D, Dv);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "qkv_store: page size %d is not a power of two", page_size);
    XR_REQUIRE(Hk == 0 || (k_cache && v_cache && k && v && block_table), "qkv_store: keys and values need their cache and table");
    if (T == 0) return XR_OK;
    if (dtype == XR_F32)
        k_qkv_store<float><<<T, 256, 0, stream>>>((float*)q_out, (float*)k_cache, (float*)v_cache, q, k, v, ld, positions,
                                                  req_of_token, block_table, table_stride, H * D, Hk, D, Dv, shift,
                                                  page_size - 1, page_size);
    else if (dtype == XR_BF16)
        k_qkv_store<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)q_out, (bf16_t*)k_cache, (bf16_t*)v_cache, q, k, v, ld, positions,
                                                   req_of_token, block_table, table_stride, H * D, Hk, D, Dv, shift,
                                                   page_size - 1, page_size);
    else { xr_set_error("qkv_store: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("qkv_store");
    return XR_OK;
}

// ---------------------------------------------------------------- a norm of every query and key head
// In place on the 32-bit projections, between the product and the store: every head of D channels is divided
// by its root mean square (eps inside the root) and multiplied by a weight over D that the heads share (one for
// the queries, one for the keys; either may be absent: that side is left alone).  With `every` > 0 the queries
// of the token at position p are also multiplied by 1 + coef * ln(floor((p + 1) / every) + 1): queries far
// into a sequence are sharpened.  A wave a head.
__global__ __launch_bounds__(256) void k_head_rmsnorm(float* __restrict__ q, float* __restrict__ k, int ld,
                                                      const float* __restrict__ wq, const float* __restrict__ wk,
                                                      const int* __restrict__ positions, int H, int Hk, int D, float eps,
                                                      float coef, int every) {
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (head >= H + Hk) return;
    const bool is_q = head < H;
    const float* w = is_q ? wq : wk;
    float temp = 1.f;
    if (is_q && every > 0) temp = 1.0f + coef * logf((float)((positions[t] + 1) / every + 1));
    if (!w && temp == 1.f) return;
    float* x = (is_q ? q + (size_t)head * D : k + (size_t)(head - H) * D) + (size_t)t * ld;
    float f = temp;
    if (w) {
        float ss = 0.f;
        for (int d = lane; d < D; d += 64) ss = fmaf(x[d], x[d], ss);
        f *= 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    }
    for (int d = lane; d < D; d += 64) x[d] = x[d] * f * (w ? w[d] : 1.f);
}

extern "C" int xr_head_rmsnorm(float* q, float* k, int ld, const float* wq, const float* wk, const int* positions, int T,
                               int H, int Hk, int D, float eps, float coef, int every, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H >= 0 && Hk >= 0 && D > 0, "head_rmsnorm: bad sizes T=%d H=%d Hk=%d D=%d", T, H, Hk, D);
    XR_REQUIRE((H == 0 || q) && (Hk == 0 || k), "head_rmsnorm: heads without their rows");
    XR_REQUIRE(every >= 0 && (every == 0 || positions), "head_rmsnorm: a temperature every %d positions needs the positions", every);
    XR_REQUIRE(eps >= 0.f, "head_rmsnorm: eps %g is negative", eps);
    if (T == 0 || H + Hk == 0) return XR_OK;
    k_head_rmsnorm<<<dim3(T, (H + Hk + 3) / 4), 256, 0, stream>>>(q, k, ld, wq, wk, positions, H, Hk, D, eps, coef, every);
    XR_CHECK_LAUNCH("head_rmsnorm");
    return XR_OK;
}

// ---------------------------------------------------------------- the means of the blocks a step completes
// Request b held starts[b] positions before the step and brings n = cu_q[b+1] - cu_q[b]: the
// blocks starts[b] / P .. (starts[b] + n) / P - 1 are complete now.  One workgroup per
// (new block, kv head, request); blocks that do not exist leave at once.
template <typename T>
__global__ __launch_bounds__(256) void k_pool_blocks(T* __restrict__ pk, T* __restrict__ pv, const T* __restrict__ kc,
                                                    const T* __restrict__ vc, const int* __restrict__ starts,
                                                    const int* __restrict__ cu_q, const int* __restrict__ block_table,
                                                    int table_stride, const int* __restrict__ pool_table, int pool_stride,
                                                    int Hk, int D, int Dv, int P, int page_shift, int page_mask, int page_size) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int s = starts[b], n = cu_q[b + 1] - cu_q[b];
    const int blk = s / P + blockIdx.x;
    if (blk >= (s + n) / P) return;
    const int* bt = block_table + (size_t)b * table_stride;
    const int ppage = pool_table[(size_t)b * pool_stride + (blk >> page_shift)];
    const int poff = blk & page_mask;
    const float inv = 1.0f / (float)P;
    // channels of the key, then channels of the value, a thread each; positions in ascending order
    for (int e = threadIdx.x; e < D + Dv; e += 256) {
        float acc = 0.f;
        if (e < D) {
            for (int j = 0; j < P; ++j) {
                const int pos = blk * P + j;
                acc += ld<T>(kc, (((size_t)bt[pos >> page_shift] * Hk + h) * page_size + (pos & page_mask)) * D + e);
            }
            st<T>(pk, (((size_t)ppage * Hk + h) * page_size + poff) * D + e, acc * inv);
        } else {
            const int d = e - D;
            for (int j = 0; j < P; ++j) {
                const int pos = blk * P + j;
                acc += ld<T>(vc, (((size_t)bt[pos >> page_shift] * Hk + h) * Dv + d) * page_size + (pos & page_mask));
            }
            st<T>(pv, (((size_t)ppage * Hk + h) * Dv + d) * page_size + poff, acc * inv);
        }
    }
}

extern "C" int xr_pool_blocks(void* pk, void* pv, const void* k_cache, const void* v_cache, const int* starts,
                              const int* cu_q, const int* block_table, int table_stride, const int* pool_table,
                              int pool_stride, int B, int max_new_blocks, int Hk, int D, int Dv, int P, int page_size,
                              int dtype, hipStream_t stream) {
    XR_REQUIRE(B >= 0 && Hk > 0 && D > 0 && Dv > 0 && P > 0, "pool_blocks: bad sizes B=%d Hk=%d D=%d Dv=%d P=%d", B, Hk, D, Dv, P);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "pool_blocks: page size %d is not a power of two", page_size);
    if (B == 0 || max_new_blocks <= 0) return XR_OK;
    dim3 grid(max_new_blocks, Hk, B);
    if (dtype == XR_F32)
        k_pool_blocks<float><<<grid, 256, 0, stream>>>((float*)pk, (float*)pv, (const float*)k_cache, (const float*)v_cache,
                                                      starts, cu_q, block_table, table_stride, pool_table, pool_stride, Hk,
                                                      D, Dv, P, shift, page_size - 1, page_size);
    else if (dtype == XR_BF16)
        k_pool_blocks<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)pk, (bf16_t*)pv, (const bf16_t*)k_cache,
                                                       (const bf16_t*)v_cache, starts, cu_q, block_table, table_stride,
                                                       pool_table, pool_stride, Hk, D, Dv, P, shift, page_size - 1, page_size);
    else { xr_set_error("pool_blocks: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("pool_blocks");
    return XR_OK;
}

// ---------------------------------------------------------------- the attention itself
// One wave per (token, query head): 64 keys at a time, a lane a key for the scores, a lane a
// channel (and every 64th after it) for the values, with a running maximum and sum.
struct PoolAttnArgs {
    const int* positions;
    const int* req_of_token;
    const int* block_table;
    const int* pool_table;
    int table_stride, pool_stride;
    int H, Hk, D, Dv, page_shift, page_mask, page_size;
    float scale;
    int size, P;
};

// VEC (bfloat16, key size a multiple of 8, pages of at least 8): a key's channels are read eight at
// a time, and the values, which lie position by position inside a page, eight positions of a
// channel at a time; tiles then begin on multiples of 8 (keys below `lo` in the first tile count as
// absent), so a group of eight never leaves its page.
__device__ inline void unpack8(uint4 w, float* f) {
    f[0] = __uint_as_float(w.x << 16); f[1] = __uint_as_float(w.x & 0xffff0000u);
    f[2] = __uint_as_float(w.y << 16); f[3] = __uint_as_float(w.y & 0xffff0000u);
    f[4] = __uint_as_float(w.z << 16); f[5] = __uint_as_float(w.z & 0xffff0000u);
    f[6] = __uint_as_float(w.w << 16); f[7] = __uint_as_float(w.w & 0xffff0000u);
}

template <typename T, bool VEC>
__device__ inline void attend_range(const T* __restrict__ kc, const T* __restrict__ vc, const int* __restrict__ bt, int lo,
                                    int hi, const float* qs, int kvh, const PoolAttnArgs& a, float& m, float& l,
                                    float* acc, int lane) {
    for (int k0 = VEC ? (lo & ~7) : lo; k0 < hi; k0 += 64) {
        const int key = k0 + lane;
        const bool valid = key >= lo && key < hi;
        float s = -INFINITY;
        if (valid) {
            const T* kr = kc + (((size_t)bt[key >> a.page_shift] * a.Hk + kvh) * a.page_size + (key & a.page_mask)) * a.D;
            float dot = 0.f;
            if (VEC) {
                for (int d = 0; d < a.D; d += 8) {
                    float f[8];
                    unpack8(*reinterpret_cast<const uint4*>(kr + d), f);
#pragma unroll
                    for (int i = 0; i < 8; ++i) dot = fmaf(qs[d + i], f[i], dot);
                }
            } else {
                for (int d = 0; d < a.D; ++d) dot = fmaf(qs[d], ld<T>(kr, d), dot);
            }
            s = dot * a.scale;
        }
        const float mn = fmaxf(m, wave_max(s));
        const float p = valid ? expf(s - mn) : 0.f;
        const float corr = mn == -INFINITY ? 1.f : expf(m - mn);
        l = l * corr + wave_sum(p);
#pragma unroll
        for (int dd = 0; dd < AP_MAX_D / 64; ++dd) acc[dd] *= corr;
        const int nk = hi - k0 < 64 ? hi - k0 : 64;
        if (VEC) {
            for (int j0 = 0; j0 < nk; j0 += 8) {
                const int kj = k0 + j0;
                if (kj + 7 < lo) continue;              // eight keys below the range: their page may be gone
                float pj[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) pj[i] = __shfl(p, j0 + i, 64);
                const T* vb = vc + ((size_t)bt[kj >> a.page_shift] * a.Hk + kvh) * a.Dv * a.page_size + (kj & a.page_mask);
#pragma unroll
                for (int dd = 0; dd < AP_MAX_D / 64; ++dd) {
                    const int d = lane + 64 * dd;
                    if (d < a.Dv) {
                        float f[8];
                        unpack8(*reinterpret_cast<const uint4*>(vb + (size_t)d * a.page_size), f);
#pragma unroll
                        for (int i = 0; i < 8; ++i)
                            if (pj[i] > 0.f) acc[dd] = fmaf(pj[i], f[i], acc[dd]);     // (what lies past the range is never multiplied)
                    }
                }
            }
        } else {
            for (int j = 0; j < nk; ++j) {
                const float pj = __shfl(p, j, 64);
                const int kj = k0 + j;
                const T* vb = vc + ((size_t)bt[kj >> a.page_shift] * a.Hk + kvh) * a.Dv * a.page_size + (kj & a.page_mask);
#pragma unroll
                for (int dd = 0; dd < AP_MAX_D / 64; ++dd) {
                    const int d = lane + 64 * dd;
                    if (d < a.Dv) acc[dd] = fmaf(pj, ld<T>(vb, (size_t)d * a.page_size), acc[dd]);
                }
            }
        }
        m = mn;
    }
}

template <typename T, bool VEC>
__global__ __launch_bounds__(64) void k_attention_pooled(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ kc,
                                                         const T* __restrict__ vc, const T* __restrict__ pk,
                                                         const T* __restrict__ pv, PoolAttnArgs a) {
    __shared__ float qs[AP_MAX_D];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int pos = a.positions[t], req = a.req_of_token[t];
    const int kvh = h / (a.H / a.Hk);
    const T* qrow = q + ((size_t)t * a.H + h) * a.D;
    for (int d = lane; d < a.D; d += 64) qs[d] = ld<T>(qrow, d);
    __syncthreads();
    float m = -INFINITY, l = 0.f;
    float acc[AP_MAX_D / 64];
#pragma unroll
    for (int dd = 0; dd < AP_MAX_D / 64; ++dd) acc[dd] = 0.f;
    const int lo = pos - a.size + 1 > 0 ? pos - a.size + 1 : 0;
    // blocks b with b P + P - 1 <= pos - size, i.e. b < (pos - size + 1) / P
    const int n_blocks = (a.P > 0 && pos - a.size + 1 > 0) ? (pos - a.size + 1) / a.P : 0;
    if (n_blocks > 0)
        attend_range<T, VEC>(pk, pv, a.pool_table + (size_t)req * a.pool_stride, 0, n_blocks, qs, kvh, a, m, l, acc, lane);
    attend_range<T, VEC>(kc, vc, a.block_table + (size_t)req * a.table_stride, lo, pos + 1, qs, kvh, a, m, l, acc, lane);
    T* orow = out + ((size_t)t * a.H + h) * a.Dv;
#pragma unroll
    for (int dd = 0; dd < AP_MAX_D / 64; ++dd) {
        const int d = lane + 64 * dd;
        if (d < a.Dv) st<T>(orow, d, acc[dd] / l);
    }
}

// ---------------------------------------------------------------- the block means alone, as a partial result
// For the matrix-core attention kernels, which take the window's keys: the same softmax pieces
// over the block means only, left where those kernels leave the partial result of a key range
// (part_o [slot][kv_head][32 rows][Dv]: the normalised output; part_ml: the maximum in units of
// log2 and the sum), so that their merge adds the two.  A record of `extras` names a block of 32
// rows (row = token x heads-in-group + head) and its slot: request, row0, slot, q0, q_len, start.
// One wave a row.
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void k_pool_partial(float* __restrict__ part_o, float* __restrict__ part_ml,
                                                      const T* __restrict__ q, const T* __restrict__ pk,
                                                      const T* __restrict__ pv, const int* __restrict__ extras,
                                                      PoolAttnArgs a) {
    __shared__ float qs[4][AP_MAX_D];
    const int* ex = extras + (size_t)(blockIdx.x >> 3) * 8;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = (blockIdx.x & 7) * 4 + wave;
    const int kvh = blockIdx.y, G = a.H / a.Hk;
    const int req = ex[0], rho = ex[1] + r, slot = ex[2], q0 = ex[3], q_len = ex[4], start = ex[5];
    const int tok = rho / G, hg = rho - tok * G;
    const bool row = tok < q_len;
    if (row) {
        const T* qrow = q + ((size_t)(q0 + tok) * a.H + kvh * G + hg) * a.D;
        for (int d = lane; d < a.D; d += 64) qs[wave][d] = ld<T>(qrow, d);
    }
    __syncthreads();
    if (!row) return;
    const int pos = start + tok;
    const int n_blocks = (a.P > 0 && pos - a.size + 1 > 0) ? (pos - a.size + 1) / a.P : 0;
    float m = -INFINITY, l = 0.f;
    float acc[AP_MAX_D / 64];
#pragma unroll
    for (int dd = 0; dd < AP_MAX_D / 64; ++dd) acc[dd] = 0.f;
    if (n_blocks > 0)
        attend_range<T, VEC>(pk, pv, a.pool_table + (size_t)req * a.pool_stride, 0, n_blocks, qs[wave], kvh, a, m, l, acc, lane);
    const size_t at = ((size_t)slot * a.Hk + kvh) * 32 + r;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int dd = 0; dd < AP_MAX_D / 64; ++dd) {
        const int d = lane + 64 * dd;
        if (d < a.Dv) part_o[at * a.Dv + d] = acc[dd] * inv;
    }
    if (lane == 0) {
        part_ml[at * 2] = m * 1.44269504f;
        part_ml[at * 2 + 1] = l;
    }
}

extern "C" int xr_attention_pool_partial(float* part_o, float* part_ml, const void* q, const void* pk, const void* pv,
                                         const int* extras, int n_extras, const int* pool_table, int pool_stride, int H,
                                         int Hk, int D, int Dv, int page_size, float scale, int size, int P, int dtype,
                                         hipStream_t stream) {
    XR_REQUIRE(n_extras >= 0 && H > 0 && Hk > 0 && H % Hk == 0, "pooled partial: %d query heads over %d key/value heads", H, Hk);
    XR_REQUIRE(D > 0 && D <= AP_MAX_D && Dv > 0 && Dv <= AP_MAX_D, "pooled partial: key size %d, value size %d (1 to %d)", D, Dv, AP_MAX_D);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "pooled partial: page size %d is not a power of two", page_size);
    XR_REQUIRE(size >= 1 && P >= 1 && part_o && part_ml && q && pk && pv && extras && pool_table, "pooled partial: an operand is missing");
    if (n_extras == 0) return XR_OK;
    PoolAttnArgs a{nullptr, nullptr, nullptr, pool_table, 0, pool_stride, H, Hk, D, Dv, shift, page_size - 1, page_size, scale, size, P};
    dim3 grid((unsigned)n_extras * 8, Hk);
    const bool vec = dtype == XR_BF16 && D % 8 == 0 && page_size >= 8;
    if (dtype == XR_F32)
        k_pool_partial<float, false><<<grid, 256, 0, stream>>>(part_o, part_ml, (const float*)q, (const float*)pk, (const float*)pv, extras, a);
    else if (dtype == XR_BF16 && vec)
        k_pool_partial<bf16_t, true><<<grid, 256, 0, stream>>>(part_o, part_ml, (const bf16_t*)q, (const bf16_t*)pk, (const bf16_t*)pv, extras, a);
    else if (dtype == XR_BF16)
        k_pool_partial<bf16_t, false><<<grid, 256, 0, stream>>>(part_o, part_ml, (const bf16_t*)q, (const bf16_t*)pk, (const bf16_t*)pv, extras, a);
    else { xr_set_error("pooled partial: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("attention_pool_partial");
    return XR_OK;
}

extern "C" int xr_attention_pooled(void* out, const void* q, const void* k_cache, const void* v_cache, const void* pk,
                                   const void* pv, const int* positions, const int* req_of_token, const int* block_table,
                                   int table_stride, const int* pool_table, int pool_stride, int T, int H, int Hk, int D,
                                   int Dv, int page_size, float scale, int size, int P, int dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && H > 0 && Hk > 0 && H % Hk == 0, "pooled attention: %d query heads over %d key/value heads", H, Hk);
    XR_REQUIRE(D > 0 && D <= AP_MAX_D && Dv > 0 && Dv <= AP_MAX_D, "pooled attention: key size %d, value size %d (1 to %d)", D, Dv, AP_MAX_D);
    const int shift = ilog2_exact(page_size);
    XR_REQUIRE(shift >= 0, "pooled attention: page size %d is not a power of two", page_size);
    XR_REQUIRE(size >= 1 && P >= 0, "pooled attention: window %d, block %d", size, P);
    XR_REQUIRE(P == 0 || (pk && pv && pool_table), "pooled attention: blocks of %d need their cache and table", P);
    if (T == 0) return XR_OK;
    PoolAttnArgs a{positions, req_of_token, block_table, pool_table, table_stride, pool_stride, H, Hk, D, Dv, shift,
                   page_size - 1, page_size, scale, size, P};
    dim3 grid(T, H);
    const bool vec = dtype == XR_BF16 && D % 8 == 0 && page_size >= 8;
    if (dtype == XR_F32)
        k_attention_pooled<float, false><<<grid, 64, 0, stream>>>((float*)out, (const float*)q, (const float*)k_cache,
                                                                  (const float*)v_cache, (const float*)pk, (const float*)pv, a);
    else if (dtype == XR_BF16 && vec)
        k_attention_pooled<bf16_t, true><<<grid, 64, 0, stream>>>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                                                  (const bf16_t*)v_cache, (const bf16_t*)pk, (const bf16_t*)pv, a);
    else if (dtype == XR_BF16)
        k_attention_pooled<bf16_t, false><<<grid, 64, 0, stream>>>((bf16_t*)out, (const bf16_t*)q, (const bf16_t*)k_cache,
                                                                   (const bf16_t*)v_cache, (const bf16_t*)pk, (const bf16_t*)pv, a);
    else { xr_set_error("pooled attention: bad dtype %d", dtype); return XR_BAD_ARG; }
    XR_CHECK_LAUNCH("attention_pooled");
    return XR_OK;
}
