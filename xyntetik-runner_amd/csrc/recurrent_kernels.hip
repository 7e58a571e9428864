// Linear recurrences over time with a matrix of state per request and head, in 32-bit floats:
//
//   retention:   S <- decay_h S + k v^T;                            o = S^T q
//   delta rule:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   wkv:         o = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T    (the read-out comes before the update and
//                gives the token itself a weight u of its own; w = exp(-exp(x)) is a decay a token, head and key
//                channel, made here from x as the rows are fetched)
//   gla:         S <- diag(w) S + k v^T;                            o = S^T q    (w a decay a token, head and key
//                channel, given as it is: "gated linear attention")
//   delta rule with a decay a key channel:  S <- diag(w) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// S is [D, Dv] and its columns never meet: column c only needs v[c].  A group of R adjacent lanes
// owns one column (lane r the rows r, r+R, r+2R, ...), keeps it in registers over the whole
// portion, and the two sums over D are a few fused multiply-adds and a sum over the group's lanes
// (by lane permutes of the vector unit, no trip to LDS) a token.  R is 16 for key sizes above 32
// (a token then costs a lane 3 D / 16 multiply-adds; the recurrence is a chain, so what a token
// costs one lane is what the portion costs), else 4.  A workgroup of 256 lanes owns 256 / R
// columns of one (request, head); queries and keys of a few tokens at a time are staged in LDS,
// the rows of a lane side by side so that they are read four at a time.  The same kernel runs a
// prompt's portion and a decoded token (a portion of one).
//
// State in memory: [slot][head][J = ceil(D/R)][Dv][R], i.e. S[R j + r][c] at ((j * Dv) + c) * R + r:
// a wave's loads and stores are contiguous.  Rows past D (when D is no multiple of R) stay zero.
#include "common.h"

#define REC_TOKENS 16        // tokens staged at a time
#define XR_REC_RETENTION 0
#define XR_REC_DELTA 1
#define XR_REC_WKV 2
#define XR_REC_GLA 3
#define XR_REC_DELTA_CH 4

static inline int rec_lanes(int D) { return D > 32 ? 16 : 4; }

struct RecArgs {
    float* out;              // [T, H, Dv]
    const float* q;          // [T, ld] at the first query head; G heads of D
    const float* k;
    const float* v;          // H heads of Dv
    const float* beta;       // [T, ld_g] at head 0 (delta rule)
    const float* gate;       // [T, ld_g] at head 0: the decay of every token and head (delta rule); wkv: x of the decay, H heads of D;
                             // gla and the delta rule with channel decays: the decays themselves, H heads of D
    const float* decay;      // [H] (retention); wkv: the bonus u [H, D]
    float* state;
    const int* cu_q;
    const int* slots;
    int H, G, D, Dv, ld, ld_g;   // row strides of q/k/v and of the gate
    int ld_b;                    // row stride of beta
    // Retention over a long portion, cut into chunks of chunk_len rows that run side by side (its decay is
    // one number a head, so S_t = (the chunk's own sum from zero) + decay^(i+1) x (the state before the
    // chunk), i the row's place in the chunk):
    //   pass 1: every chunk runs the recurrence from zero (the first from the request's state), writes its
    //           read-outs and leaves its last state in scratch [request x chunk][head][J][Dv][R];
    //   k_retention_carry turns those into every chunk's true first state, and the request's new state;
    //   pass 2: every chunk but the first runs again from its true first state with nothing written
    //           (v = 0: the state just decays) and adds its read-outs to those of pass 1.
    // pass 0: one workgroup runs the whole portion.
    int pass, chunk_len, n_chunks;
    float* scratch;
    int act;                 // 1: q, k and v pass SiLU as they are fetched (0: they are taken as they are)
    // wkv in chunks: its decay is a number a token and key channel, so the state before a chunk enters the
    // chunk's last state through the product of the chunk's decays, channel by channel: pass 1 leaves that
    // product in prod [request x chunk][head][J][R] (row R j + r at j R + r) beside the chunk's last state;
    // pass 2 runs with v = 0, so that the state only decays and the bonus term is nothing.
    float* prod;
    float q_scale, k_scale;  // factors on the queries and on the keys as they are fetched (behind the activation, if there is one)
};

// the value of lane (l ^ 1), (l ^ 2) of a quad, or of the lane 4 / 8 further round a row of 16
template <int CTRL> __device__ inline float lane_permute(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}
template <int R> __device__ inline float group_sum(float v) {
    if (R >= 16) {
        v += lane_permute<0x128>(v);     // row_ror:8
        v += lane_permute<0x124>(v);     // row_ror:4
    }
    v += lane_permute<0x4E>(v);          // quad_perm [2,3,0,1]
    v += lane_permute<0xB1>(v);          // quad_perm [1,0,3,2]
    return v;
}

template <int MODE, int R, int DPER>
__global__ __launch_bounds__(256) void k_recurrence(RecArgs a) {
    constexpr int COLS = 256 / R;
    __shared__ float4 qs[REC_TOKENS][R * DPER / 4];        // [token][r * (DPER/4) + j/4] as lanes read them
    __shared__ float4 ks[REC_TOKENS][R * DPER / 4];
    constexpr bool CHD = MODE == XR_REC_WKV || MODE == XR_REC_GLA || MODE == XR_REC_DELTA_CH;      // a decay a key channel
    constexpr bool CHAIN = MODE == XR_REC_DELTA || MODE == XR_REC_DELTA_CH;                         // a chain that cannot be cut into chunks
    __shared__ float4 ws[CHD ? REC_TOKENS : 1][R * DPER / 4];      // the decays a key channel, as the keys lie
    __shared__ float vs[REC_TOKENS][COLS];
    __shared__ float bs[REC_TOKENS], gs[REC_TOKENS];
    const int h = blockIdx.y, tid = threadIdx.x;
    const int cl = tid / R, r = tid % R;
    const int col = blockIdx.x * COLS + cl;
    const bool live = col < a.Dv;
    const int pass = !CHAIN ? a.pass : 0;
    int b = blockIdx.z, chunk = 0;
    if (pass) { chunk = b % a.n_chunks; b /= a.n_chunks; }
    int row0 = a.cu_q[b], n = a.cu_q[b + 1] - row0;
    if (pass) {
        if (chunk * a.chunk_len >= n || (pass == 2 && chunk == 0)) return;
        row0 += chunk * a.chunk_len;
        n = n - chunk * a.chunk_len < a.chunk_len ? n - chunk * a.chunk_len : a.chunk_len;
    }
    if (n <= 0) return;
    const int kvh = h / (a.H / a.G);
    const int J = (a.D + R - 1) / R;
    float* sp = a.state + (((size_t)a.slots[b] * a.H + h) * J) * a.Dv * R;
    float* cp = pass ? a.scratch + ((((size_t)b * a.n_chunks + chunk) * a.H + h) * J) * a.Dv * R : nullptr;
    const float* from = pass == 2 ? cp : (pass == 1 && chunk > 0) ? nullptr : sp;
    float S[DPER];
#pragma unroll
    for (int j = 0; j < DPER; ++j) S[j] = (live && j < J && from) ? from[((size_t)j * a.Dv + col) * R + r] : 0.f;
    const float dec = MODE == XR_REC_RETENTION ? a.decay[h] : 1.f;
    float* qf = reinterpret_cast<float*>(&qs[0][0]);
    float* kf = reinterpret_cast<float*>(&ks[0][0]);
    float* wf = reinterpret_cast<float*>(&ws[0][0]);
    float ub[DPER];                 // (wkv) the bonus of this lane's rows
    float wp[(MODE == XR_REC_WKV || MODE == XR_REC_GLA) ? DPER : 1];        // (pass 1) the product of the chunk's decays of this lane's rows
#pragma unroll
    for (int j = 0; j < DPER; ++j) ub[j] = (MODE == XR_REC_WKV && R * j + r < a.D) ? a.decay[(size_t)h * a.D + R * j + r] : 0.f;
    if (MODE == XR_REC_WKV || MODE == XR_REC_GLA) {
#pragma unroll
        for (int j = 0; j < DPER; ++j) wp[j] = 1.f;
    }

    // A chunk's queries, keys, values and gates go from memory into registers while the chunk before
    // it is computed, and from there into LDS: the chain of tokens never waits for memory.
    constexpr int NQ = REC_TOKENS * R * DPER / 256;       // staged elements of q (and of k) a lane
    constexpr int NV = (REC_TOKENS * COLS + 255) / 256;
    float rq[NQ], rk[NQ], rw[CHD ? NQ : 1], rv[NV], rb = 0.f, rg = 0.f;
    auto fetch = [&](int c0) {
        const int nt = n - c0 < REC_TOKENS ? n - c0 : REC_TOKENS;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = tid + i * 256;
            const int tt = idx / (R * DPER), e = idx - tt * R * DPER;
            const int rr = e / DPER, j = e - rr * DPER, d = R * j + rr;
            const bool ok = tt < nt && d < a.D;
            const size_t row = (size_t)(row0 + c0 + (ok ? tt : 0)) * a.ld + (size_t)kvh * a.D + (ok ? d : 0);
            rq[i] = ok ? a.q[row] : 0.f;
            rk[i] = ok ? a.k[row] : 0.f;
            if (a.act) { rq[i] = rq[i] / (1.0f + expf(-rq[i])); rk[i] = rk[i] / (1.0f + expf(-rk[i])); }
            rq[i] *= a.q_scale;
            rk[i] *= a.k_scale;
            if (MODE == XR_REC_WKV)
                rw[i] = ok ? expf(-expf(a.gate[(size_t)(row0 + c0 + tt) * a.ld_g + (size_t)h * a.D + d])) : 0.f;
            if (MODE == XR_REC_GLA || MODE == XR_REC_DELTA_CH)
                rw[i] = ok ? a.gate[(size_t)(row0 + c0 + tt) * a.ld_g + (size_t)h * a.D + d] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = tid + i * 256;
            const int tt = idx / COLS, c = idx - tt * COLS;
            const int cc = blockIdx.x * COLS + c;
            const bool ok = idx < REC_TOKENS * COLS && tt < nt && cc < a.Dv && pass != 2;
            rv[i] = ok ? a.v[(size_t)(row0 + c0 + tt) * a.ld + (size_t)h * a.Dv + cc] : 0.f;
            if (a.act) rv[i] = rv[i] / (1.0f + expf(-rv[i]));
        }
        if (CHAIN && tid < nt) {
            rb = a.beta[(size_t)(row0 + c0 + tid) * a.ld_b + h];
            if (MODE == XR_REC_DELTA) rg = a.gate[(size_t)(row0 + c0 + tid) * a.ld_g + h];
        }
    };
    fetch(0);
    float4 qp[DPER / 4];            // (delta rule) the query of the token before, whose read-out is still owed
#pragma unroll
    for (int j = 0; j < DPER / 4; ++j) qp[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    int prev_row = -1;
    for (int c0 = 0; c0 < n; c0 += REC_TOKENS) {
        const int nt = n - c0 < REC_TOKENS ? n - c0 : REC_TOKENS;
        __syncthreads();
        // element d = R j + rr of a token goes to place rr * DPER + j; places past D hold zero
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            qf[tid + i * 256] = rq[i]; kf[tid + i * 256] = rk[i];
            if (CHD) wf[tid + i * 256] = rw[i];
        }
#pragma unroll
        for (int i = 0; i < NV; ++i)
            if (tid + i * 256 < REC_TOKENS * COLS) (&vs[0][0])[tid + i * 256] = rv[i];
        if (CHAIN && tid < REC_TOKENS) { bs[tid] = rb; gs[tid] = rg; }
        __syncthreads();
        if (c0 + REC_TOKENS < n) fetch(c0 + REC_TOKENS);
        if (MODE == XR_REC_DELTA_CH) {
            // As below, with a decay of its own for every row of the state: the decayed state's S^T k is a sum
            // over S w k, and the update scales every row by its own w.
            for (int tt = 0; tt < nt; ++tt) {
                const float4* kq = &ks[tt][r * (DPER / 4)];
                const float4* qq = &qs[tt][r * (DPER / 4)];
                const float4* wq = &ws[tt][r * (DPER / 4)];
                const float vv = vs[tt][cl], bt = bs[tt];
                float4 kk[DPER / 4], w4[DPER / 4];
                float d0 = 0.f, d1 = 0.f, p0 = 0.f, p1 = 0.f;
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    kk[j >> 2] = kq[j >> 2];
                    w4[j >> 2] = wq[j >> 2];
                    d0 = fmaf(S[j] * w4[j >> 2].x, kk[j >> 2].x, d0); d1 = fmaf(S[j + 1] * w4[j >> 2].y, kk[j >> 2].y, d1);
                    d0 = fmaf(S[j + 2] * w4[j >> 2].z, kk[j >> 2].z, d0); d1 = fmaf(S[j + 3] * w4[j >> 2].w, kk[j >> 2].w, d1);
                    p0 = fmaf(S[j], qp[j >> 2].x, p0); p1 = fmaf(S[j + 1], qp[j >> 2].y, p1);
                    p0 = fmaf(S[j + 2], qp[j >> 2].z, p0); p1 = fmaf(S[j + 3], qp[j >> 2].w, p1);
                }
                const float dsum = group_sum<R>(d0 + d1), psum = group_sum<R>(p0 + p1);
                if (prev_row >= 0 && live && r == 0) a.out[((size_t)prev_row * a.H + h) * a.Dv + col] = psum;
                const float u = bt * (vv - dsum);
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    S[j] = fmaf(w4[j >> 2].x, S[j], kk[j >> 2].x * u); S[j + 1] = fmaf(w4[j >> 2].y, S[j + 1], kk[j >> 2].y * u);
                    S[j + 2] = fmaf(w4[j >> 2].z, S[j + 2], kk[j >> 2].z * u); S[j + 3] = fmaf(w4[j >> 2].w, S[j + 3], kk[j >> 2].w * u);
                    qp[j >> 2] = qq[j >> 2];
                }
                prev_row = row0 + c0 + tt;
            }
        } else if (MODE == XR_REC_DELTA) {
            // The state's chain a token is: sum over the column (S . k), u, one multiply-add.  The
            // read-out (S . q) is off that chain but a wave issues in order, so the read-out of the
            // token before runs in the same pass over S as this token's sum: two chains side by side.
            for (int tt = 0; tt < nt; ++tt) {
                const float4* kq = &ks[tt][r * (DPER / 4)];
                const float4* qq = &qs[tt][r * (DPER / 4)];
                const float vv = vs[tt][cl], g = gs[tt], bt = bs[tt];
                float4 kk[DPER / 4];
                float d0 = 0.f, d1 = 0.f, p0 = 0.f, p1 = 0.f;
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    kk[j >> 2] = kq[j >> 2];
                    d0 = fmaf(S[j], kk[j >> 2].x, d0); d1 = fmaf(S[j + 1], kk[j >> 2].y, d1);
                    d0 = fmaf(S[j + 2], kk[j >> 2].z, d0); d1 = fmaf(S[j + 3], kk[j >> 2].w, d1);
                    p0 = fmaf(S[j], qp[j >> 2].x, p0); p1 = fmaf(S[j + 1], qp[j >> 2].y, p1);
                    p0 = fmaf(S[j + 2], qp[j >> 2].z, p0); p1 = fmaf(S[j + 3], qp[j >> 2].w, p1);
                }
                const float dsum = group_sum<R>(d0 + d1), psum = group_sum<R>(p0 + p1);
                if (prev_row >= 0 && live && r == 0) a.out[((size_t)prev_row * a.H + h) * a.Dv + col] = psum;
                const float u = bt * (vv - g * dsum);          // S^T k of the decayed state = g (S^T k)
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    S[j] = fmaf(g, S[j], kk[j >> 2].x * u); S[j + 1] = fmaf(g, S[j + 1], kk[j >> 2].y * u);
                    S[j + 2] = fmaf(g, S[j + 2], kk[j >> 2].z * u); S[j + 3] = fmaf(g, S[j + 3], kk[j >> 2].w * u);
                    qp[j >> 2] = qq[j >> 2];
                }
                prev_row = row0 + c0 + tt;
            }
        } else if (MODE == XR_REC_WKV || MODE == XR_REC_GLA) {
            // The chain is one multiply-add a token, as retention's; the read-out is of the state before the
            // update plus the token's own k v^T times the bonus.  Four tokens' read-outs run side by side.
            auto token = [&](int tt) {
                const float4* kq = &ks[tt][r * (DPER / 4)];
                const float4* qq = &qs[tt][r * (DPER / 4)];
                const float4* wq = &ws[tt][r * (DPER / 4)];
                const float vv = vs[tt][cl];
                float o0 = 0.f, o1 = 0.f;
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    const float4 kk = kq[j >> 2], q4 = qq[j >> 2], w4 = wq[j >> 2];
                    const float t0 = kk.x * vv, t1 = kk.y * vv, t2 = kk.z * vv, t3 = kk.w * vv;
                    if (MODE == XR_REC_WKV) {
                        o0 = fmaf(q4.x, fmaf(ub[j], t0, S[j]), o0); o1 = fmaf(q4.y, fmaf(ub[j + 1], t1, S[j + 1]), o1);
                        o0 = fmaf(q4.z, fmaf(ub[j + 2], t2, S[j + 2]), o0); o1 = fmaf(q4.w, fmaf(ub[j + 3], t3, S[j + 3]), o1);
                    }
                    S[j] = fmaf(w4.x, S[j], t0); S[j + 1] = fmaf(w4.y, S[j + 1], t1);
                    S[j + 2] = fmaf(w4.z, S[j + 2], t2); S[j + 3] = fmaf(w4.w, S[j + 3], t3);
                    if (MODE == XR_REC_GLA) {       // the read-out sees the token's own write
                        o0 = fmaf(q4.x, S[j], o0); o1 = fmaf(q4.y, S[j + 1], o1);
                        o0 = fmaf(q4.z, S[j + 2], o0); o1 = fmaf(q4.w, S[j + 3], o1);
                    }
                    if (pass == 1) { wp[j] *= w4.x; wp[j + 1] *= w4.y; wp[j + 2] *= w4.z; wp[j + 3] *= w4.w; }
                }
                return o0 + o1;
            };
            int tt = 0;
            for (; tt + 4 <= nt; tt += 4) {
                float oo[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) oo[x] = token(tt + x);
#pragma unroll
                for (int x = 0; x < 4; ++x) oo[x] = group_sum<R>(oo[x]);
                if (live && r == 0) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        float* dst = a.out + ((size_t)(row0 + c0 + tt + x) * a.H + h) * a.Dv + col;
                        *dst = pass == 2 ? *dst + oo[x] : oo[x];
                    }
                }
            }
            for (; tt < nt; ++tt) {
                const float o = group_sum<R>(token(tt));
                if (live && r == 0) {
                    float* dst = a.out + ((size_t)(row0 + c0 + tt) * a.H + h) * a.Dv + col;
                    *dst = pass == 2 ? *dst + o : o;
                }
            }
        } else {
            // Retention's chain is one multiply-add a token; four tokens' read-outs run side by side.
            int tt = 0;
            for (; tt + 4 <= nt; tt += 4) {
                float oo[4];
#pragma unroll
                for (int x = 0; x < 4; ++x) {
                    const float4* kq = &ks[tt + x][r * (DPER / 4)];
                    const float4* qq = &qs[tt + x][r * (DPER / 4)];
                    const float vv = vs[tt + x][cl];
                    float o0 = 0.f, o1 = 0.f;
#pragma unroll
                    for (int j = 0; j < DPER; j += 4) {
                        const float4 kk = kq[j >> 2], q4 = qq[j >> 2];
                        S[j] = fmaf(dec, S[j], kk.x * vv); S[j + 1] = fmaf(dec, S[j + 1], kk.y * vv);
                        S[j + 2] = fmaf(dec, S[j + 2], kk.z * vv); S[j + 3] = fmaf(dec, S[j + 3], kk.w * vv);
                        o0 = fmaf(S[j], q4.x, o0); o1 = fmaf(S[j + 1], q4.y, o1);
                        o0 = fmaf(S[j + 2], q4.z, o0); o1 = fmaf(S[j + 3], q4.w, o1);
                    }
                    oo[x] = o0 + o1;
                }
#pragma unroll
                for (int x = 0; x < 4; ++x) oo[x] = group_sum<R>(oo[x]);
                if (live && r == 0) {
#pragma unroll
                    for (int x = 0; x < 4; ++x) {
                        float* dst = a.out + ((size_t)(row0 + c0 + tt + x) * a.H + h) * a.Dv + col;
                        *dst = pass == 2 ? *dst + oo[x] : oo[x];
                    }
                }
            }
            for (; tt < nt; ++tt) {
                const float4* kq = &ks[tt][r * (DPER / 4)];
                const float4* qq = &qs[tt][r * (DPER / 4)];
                const float vv = vs[tt][cl];
                float o0 = 0.f, o1 = 0.f;
#pragma unroll
                for (int j = 0; j < DPER; j += 4) {
                    const float4 kk = kq[j >> 2], q4 = qq[j >> 2];
                    S[j] = fmaf(dec, S[j], kk.x * vv); S[j + 1] = fmaf(dec, S[j + 1], kk.y * vv);
                    S[j + 2] = fmaf(dec, S[j + 2], kk.z * vv); S[j + 3] = fmaf(dec, S[j + 3], kk.w * vv);
                    o0 = fmaf(S[j], q4.x, o0); o1 = fmaf(S[j + 1], q4.y, o1);
                    o0 = fmaf(S[j + 2], q4.z, o0); o1 = fmaf(S[j + 3], q4.w, o1);
                }
                const float o = group_sum<R>(o0 + o1);
                if (live && r == 0) {
                    float* dst = a.out + ((size_t)(row0 + c0 + tt) * a.H + h) * a.Dv + col;
                    *dst = pass == 2 ? *dst + o : o;
                }
            }
        }
    }
    if (CHAIN) {      // the last token's read-out
        float p0 = 0.f, p1 = 0.f;
#pragma unroll
        for (int j = 0; j < DPER; j += 4) {
            p0 = fmaf(S[j], qp[j >> 2].x, p0); p1 = fmaf(S[j + 1], qp[j >> 2].y, p1);
            p0 = fmaf(S[j + 2], qp[j >> 2].z, p0); p1 = fmaf(S[j + 3], qp[j >> 2].w, p1);
        }
        const float psum = group_sum<R>(p0 + p1);
        if (prev_row >= 0 && live && r == 0) a.out[((size_t)prev_row * a.H + h) * a.Dv + col] = psum;
    }
    if (live && pass != 2) {
        float* to = pass == 1 ? cp : sp;
#pragma unroll
        for (int j = 0; j < DPER; ++j)
            if (j < J) to[((size_t)j * a.Dv + col) * R + r] = S[j];
    }
    if ((MODE == XR_REC_WKV || MODE == XR_REC_GLA) && pass == 1 && col == 0) {      // every column holds the same products: the first writes them
        float* pp = a.prod + (((size_t)b * a.n_chunks + chunk) * a.H + h) * J * R;
#pragma unroll
        for (int j = 0; j < DPER; ++j)
            if (j < J) pp[j * R + r] = wp[j];
    }
}

// Between the two passes over the chunks: scratch[b][c] holds chunk c's last state as if it had begun at
// zero (chunk 0's is true).  In place, chunk by chunk: the true first state of chunk c (for pass 2), and
// at the end the request's new state.  One thread an element of a head's state.
template <bool WKV>
__global__ __launch_bounds__(256) void k_retention_carry(RecArgs a, int per_head, int R) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= per_head) return;
    const int n = a.cu_q[b + 1] - a.cu_q[b];
    if (n <= 0) return;
    const int nc = (n + a.chunk_len - 1) / a.chunk_len;
    const float dec = WKV ? 1.f : a.decay[h];
    const size_t step = (size_t)a.H * per_head;
    float* cp = a.scratch + ((size_t)b * a.n_chunks * a.H + h) * per_head + e;
    // (wkv) element e = (j Dv + c) R + r of the state is row R j + r, whose product lies at j R + r
    const int JR = per_head / a.Dv;
    const float* pp = WKV ? a.prod + ((size_t)b * a.n_chunks * a.H + h) * JR + (e / (a.Dv * R)) * R + e % R : nullptr;
    float t = cp[0];
    for (int c = 1; c < nc; ++c) {
        const int len = n - c * a.chunk_len < a.chunk_len ? n - c * a.chunk_len : a.chunk_len;
        const float own = cp[c * step];
        cp[c * step] = t;
        t = fmaf(WKV ? pp[(size_t)c * a.H * JR] : powf(dec, (float)len), t, own);
    }
    a.state[((size_t)a.slots[b] * a.H + h) * per_head + e] = t;
}

// the shape of a request's state as [H, shape[0], Dv, shape[1]]
extern "C" int xr_recurrence_state_dims(int D, int* rows, int* lanes) {
    *lanes = rec_lanes(D);
    *rows = (D + *lanes - 1) / *lanes;
    return XR_OK;
}

extern "C" int xr_linear_recurrence(float* out, const float* q, const float* k, const float* v, const float* beta,
                                    const float* gate, const float* decay, float* state, const int* cu_q,
                                    const int* slots, int B, int H, int G, int D, int Dv, int ld, int ld_g, int ld_b, int mode,
                                    int chunk_len, int n_chunks, float* scratch, float* prod, int act, float q_scale, float k_scale,
                                    hipStream_t stream) {
    XR_REQUIRE(B >= 0 && H > 0 && G > 0 && H % G == 0, "recurrence: %d heads over %d key heads", H, G);
    XR_REQUIRE(D > 0 && D <= 256 && Dv > 0, "recurrence: key size %d (1 to 256), value size %d", D, Dv);
    XR_REQUIRE(mode >= XR_REC_RETENTION && mode <= XR_REC_DELTA_CH, "recurrence: mode %d", mode);
    const bool chain = mode == XR_REC_DELTA || mode == XR_REC_DELTA_CH;
    XR_REQUIRE(mode == XR_REC_RETENTION ? decay != nullptr : chain ? (beta != nullptr && gate != nullptr)
               : mode == XR_REC_GLA ? gate != nullptr : (gate != nullptr && decay != nullptr),
               "recurrence: the mode's gates are missing");
    XR_REQUIRE(mode != XR_REC_WKV || (G == H && ld_g >= H * D && act == 0), "recurrence: wkv has a key head a head and decays of %d x %d a row", H, D);
    XR_REQUIRE(mode != XR_REC_GLA || (G == H && ld_g >= H * D), "recurrence: gla has a key head a head and decays of %d x %d a row", H, D);
    XR_REQUIRE(mode != XR_REC_DELTA_CH || (ld_g >= H * D && ld_b >= H), "recurrence: the delta rule with channel decays needs decays of %d x %d a row", H, D);
    XR_REQUIRE(mode != XR_REC_DELTA || ld_b >= H, "recurrence: beta of %d heads a row", H);
    XR_REQUIRE(out && q && k && v && state && cu_q && slots, "recurrence: a pointer is missing");
    XR_REQUIRE(act == 0 || act == 1, "recurrence: activation %d of q, k and v (0: none, 1: SiLU)", act);
    if (B == 0) return XR_OK;
    const bool chunks = chunk_len > 0;
    XR_REQUIRE(!chunks || (!chain && n_chunks > 1 && scratch && chunk_len % REC_TOKENS == 0),
               "recurrence: chunks are for retention and wkv, with room for their states");
    XR_REQUIRE(!chunks || (mode != XR_REC_WKV && mode != XR_REC_GLA) || prod, "recurrence: channel decays in chunks need room for the chunks' decay products");
    XR_REQUIRE(!chunks || (long long)B * n_chunks <= 65535, "recurrence: %d requests of %d chunks", B, n_chunks);
    RecArgs a{out, q, k, v, beta, gate, decay, state, cu_q, slots, H, G, D, Dv, ld, ld_g, ld_b, chunks ? 1 : 0, chunk_len, n_chunks, scratch, act, prod,
              q_scale, k_scale};
    const int R = rec_lanes(D), cols = 256 / R, per = (D + R - 1) / R;
    dim3 grid((Dv + cols - 1) / cols, H, chunks ? B * n_chunks : B);
#define REC(M)                                                                          \
    do {                                                                                \
        if (R == 4) k_recurrence<M, 4, 8><<<grid, 256, 0, stream>>>(a);                 \
        else if (per <= 4) k_recurrence<M, 16, 4><<<grid, 256, 0, stream>>>(a);         \
        else if (per <= 8) k_recurrence<M, 16, 8><<<grid, 256, 0, stream>>>(a);         \
        else k_recurrence<M, 16, 16><<<grid, 256, 0, stream>>>(a);                      \
    } while (0)
    if (mode == XR_REC_DELTA) REC(XR_REC_DELTA);
    else if (mode == XR_REC_DELTA_CH) REC(XR_REC_DELTA_CH);
    else if (mode == XR_REC_WKV) REC(XR_REC_WKV);
    else if (mode == XR_REC_GLA) REC(XR_REC_GLA);
    else REC(XR_REC_RETENTION);
    if (chunks) {
        const int per_head = per * Dv * R;
        const dim3 cgrid((per_head + 255) / 256, H, B);
        if (mode == XR_REC_WKV || mode == XR_REC_GLA) k_retention_carry<true><<<cgrid, 256, 0, stream>>>(a, per_head, R);
        else k_retention_carry<false><<<cgrid, 256, 0, stream>>>(a, per_head, R);
        a.pass = 2;
        if (mode == XR_REC_WKV) REC(XR_REC_WKV);
        else if (mode == XR_REC_GLA) REC(XR_REC_GLA);
        else REC(XR_REC_RETENTION);
    }
#undef REC
    XR_CHECK_LAUNCH("linear_recurrence");
    return XR_OK;
}
