// Many small matrix products in one launch, on the matrix cores: out_g = a_g @ w_g^T for groups g
// that each have a weight matrix [N, K] of their own (bfloat16, 32-bit accumulation).
//
//   * heads:   every group has the same T rows; row t of group g is a + t * lda + g * a_group_stride
//              (a column range of a wider row), its result goes to out + t * ldo + g * o_group_stride.
//              The per-head products of latent attention (queries into the latent's space, the
//              attention's output out of it).
//   * experts: the groups' rows are listed in `perm` (group g owns perm[start .. start + count)),
//              cut into tiles by k_moe_sort; input row = perm[p] / gather_div, output row = perm[p].
//              The two products of routed experts over many tokens.
//
// A wave computes 16 * RT weight rows x 16 * MT rows with v_mfma_f32_16x16x32_bf16 (weights as the A
// operand, rows as the B operand: a lane then holds 4 consecutive output columns of one row) and
// reads its fragments straight from memory, 16 bytes a lane; the four waves of a workgroup take
// four neighbouring groups of weight rows and share the rows' fragments through the caches.
// Epilogue: nothing, or relu squared.
#include "common.h"

typedef __bf16 gm_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gm_f32x4 __attribute__((ext_vector_type(4)));

#define GM_ACT_NONE 0
#define GM_ACT_RELU2 1

struct GroupedArgs {
    const bf16_t* a;
    const bf16_t* w;
    void* out;
    long long a_group_stride, w_group_stride, o_group_stride;
    int lda, ldo, N, K, out_bf16, act;
    // experts: tiles from the sort; heads: tile_group null, tiles_per_group tiles of every group
    const int* perm;
    const int* tile_group;
    const int* tile_start;
    const int* tile_count;
    const int* n_tiles;
    int gather_div, T, tiles_per_group;
};

__device__ inline gm_bf16x8 gm_frag(const bf16_t* p, bool ok) {
    uint4 v = make_uint4(0, 0, 0, 0);
    if (ok) v = *reinterpret_cast<const uint4*>(p);
    union { uint4 u; gm_bf16x8 b; } c;
    c.u = v;
    return c.b;
}

template <int MT, int RT>
__global__ __launch_bounds__(256) void k_grouped_gemm(GroupedArgs g) {
    const int tile = blockIdx.x;
    int group, row0, rows;
    if (g.tile_group) {
        if (tile >= *g.n_tiles) return;
        group = g.tile_group[tile];
        row0 = g.tile_start[tile];
        rows = g.tile_count[tile];
    } else {
        group = tile / g.tiles_per_group;
        row0 = (tile - group * g.tiles_per_group) * (16 * MT);
        rows = g.T - row0 < 16 * MT ? g.T - row0 : 16 * MT;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int l16 = lane & 15, lq = lane >> 4;
    const int n0 = (blockIdx.y * 4 + wave) * (16 * RT);
    if (n0 >= g.N) return;

    const bf16_t* ap[MT];
    long long orow[MT];
    bool a_ok[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int r = i * 16 + l16;
        a_ok[i] = r < rows;
        int in_row, out_row;
        if (g.perm) {
            const int p = g.perm[row0 + (a_ok[i] ? r : 0)];
            in_row = p / g.gather_div;
            out_row = p;
        } else {
            in_row = out_row = row0 + (a_ok[i] ? r : 0);
        }
        ap[i] = g.a + (long long)in_row * g.lda + (long long)group * g.a_group_stride;
        orow[i] = (long long)out_row * g.ldo + (long long)group * g.o_group_stride;
    }
    const bf16_t* wp[RT];
    bool w_ok[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
        const int n = n0 + r * 16 + l16;
        w_ok[r] = n < g.N;
        wp[r] = g.w + (long long)group * g.w_group_stride + (long long)(w_ok[r] ? n : 0) * g.K;
    }
    gm_f32x4 acc[RT][MT];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[r][i] = gm_f32x4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < g.K; k0 += 64) {
        gm_bf16x8 wf[2][RT], af[2][MT];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int k = k0 + u * 32 + lq * 8;
            const bool k_ok = k < g.K;
#pragma unroll
            for (int r = 0; r < RT; ++r) wf[u][r] = gm_frag(wp[r] + k, k_ok && w_ok[r]);
#pragma unroll
            for (int i = 0; i < MT; ++i) af[u][i] = gm_frag(ap[i] + k, k_ok && a_ok[i]);
        }
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int i = 0; i < MT; ++i)
                    acc[r][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[u][r], af[u][i], acc[r][i], 0, 0, 0);
    }
    // acc[r][i][e]: output column n0 + r * 16 + 4 * (lane / 16) + e of row i * 16 + lane % 16
    const bool vec_out = g.ldo % 4 == 0 && g.o_group_stride % 4 == 0 && ((uintptr_t)g.out % 16) == 0;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        if (!a_ok[i]) continue;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int n = n0 + r * 16 + lq * 4;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = acc[r][i][e];
                if (g.act == GM_ACT_RELU2) { v[e] = fmaxf(v[e], 0.f); v[e] *= v[e]; }
            }
            if (vec_out && n + 3 < g.N) {       // the lane's 4 columns in one store
                if (g.out_bf16) {
                    uint2 w2;
                    w2.x = pack_bf16x2(v[0], v[1]);
                    w2.y = pack_bf16x2(v[2], v[3]);
                    *reinterpret_cast<uint2*>((bf16_t*)g.out + orow[i] + n) = w2;
                } else {
                    *reinterpret_cast<float4*>((float*)g.out + orow[i] + n) = make_float4(v[0], v[1], v[2], v[3]);
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e >= g.N) continue;
                if (g.out_bf16) ((bf16_t*)g.out)[orow[i] + n + e] = f32_to_bf16(v[e]);
                else ((float*)g.out)[orow[i] + n + e] = v[e];
            }
        }
    }
}

// The same product for tiles of 128 rows where the output is wide: a workgroup computes 128 rows x 128 weight
// rows, its operands staged in LDS once for all four waves (a wave takes 64 x 64 of them).  K goes in slices
// of 64: the next slice is fetched into registers (16 bytes a lane and piece, the rows of an expert gathered
// through `perm`) while the matrix cores work on the one in LDS.  Rows of LDS are 72 elements apart, so the
// 16 rows a fragment read touches do not all start in one bank.
#define GL_BM 128
#define GL_KS 64
#define GL_LD 72
template <int RT>        // groups of 16 weight rows a wave: 4 (128 weight rows a workgroup) or 8 (256)
__global__ __launch_bounds__(256) void k_grouped_gemm_lds(GroupedArgs g) {
    constexpr int GL_BN = 32 * RT, WP = RT;       // weight rows a workgroup; 16-byte pieces of them a thread copies a slice
    __shared__ __attribute__((aligned(16))) bf16_t As[GL_BM * GL_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[GL_BN * GL_LD];
    const int tile = blockIdx.x;
    int group, row0, rows;
    if (g.tile_group) {
        if (tile >= *g.n_tiles) return;
        group = g.tile_group[tile];
        row0 = g.tile_start[tile];
        rows = g.tile_count[tile];
    } else {
        group = tile / g.tiles_per_group;
        row0 = (tile - group * g.tiles_per_group) * GL_BM;
        rows = g.T - row0 < GL_BM ? g.T - row0 : GL_BM;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, lq = lane >> 4;
    const int wm = wave & 1, wn = wave >> 1;
    const int nb = blockIdx.y * GL_BN;

    // what this thread copies of a slice: 4 pieces of 16 bytes of the rows and 4 of the weights;
    // piece j is row (tid / 8) + 32 j, columns (tid % 8) * 8 .. + 8 of the slice
    const int crow = tid >> 3, ccol = (tid & 7) * 8;
    const bf16_t* a_src[4];
    const bf16_t* w_src[WP];
    bool a_on[4], w_on[WP];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int r = crow + 32 * j;
        a_on[j] = r < rows;
        const int p = g.perm ? g.perm[row0 + (a_on[j] ? r : 0)] : row0 + (a_on[j] ? r : 0);
        a_src[j] = g.a + (long long)(g.perm ? p / g.gather_div : p) * g.lda + (long long)group * g.a_group_stride + ccol;
    }
#pragma unroll
    for (int j = 0; j < WP; ++j) {
        const int n = nb + crow + 32 * j;
        w_on[j] = n < g.N;
        w_src[j] = g.w + (long long)group * g.w_group_stride + (long long)(w_on[j] ? n : 0) * g.K + ccol;
    }
    gm_f32x4 acc[RT][4];
#pragma unroll
    for (int r = 0; r < RT; ++r)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[r][i] = gm_f32x4{0.f, 0.f, 0.f, 0.f};

    uint4 ra[4], rw[WP];
    auto fetch = [&](int k0) {
        const bool k_ok = k0 + ccol < g.K;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            ra[j] = make_uint4(0, 0, 0, 0);
            if (k_ok && a_on[j]) ra[j] = *reinterpret_cast<const uint4*>(a_src[j] + k0);
        }
#pragma unroll
        for (int j = 0; j < WP; ++j) {
            rw[j] = make_uint4(0, 0, 0, 0);
            if (k_ok && w_on[j]) rw[j] = *reinterpret_cast<const uint4*>(w_src[j] + k0);
        }
    };
    fetch(0);
    for (int k0 = 0; k0 < g.K; k0 += GL_KS) {
        __syncthreads();                        // the slice before has been read by every wave
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<uint4*>(&As[(crow + 32 * j) * GL_LD + ccol]) = ra[j];
#pragma unroll
        for (int j = 0; j < WP; ++j) *reinterpret_cast<uint4*>(&Ws[(crow + 32 * j) * GL_LD + ccol]) = rw[j];
        __syncthreads();
        if (k0 + GL_KS < g.K) fetch(k0 + GL_KS);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            gm_bf16x8 wf[RT], af[4];
#pragma unroll
            for (int r = 0; r < RT; ++r) {
                union { uint4 v; gm_bf16x8 b; } c;
                c.v = *reinterpret_cast<const uint4*>(&Ws[(wn * 16 * RT + r * 16 + l16) * GL_LD + u * 32 + lq * 8]);
                wf[r] = c.b;
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                union { uint4 v; gm_bf16x8 b; } c;
                c.v = *reinterpret_cast<const uint4*>(&As[(wm * 64 + i * 16 + l16) * GL_LD + u * 32 + lq * 8]);
                af[i] = c.b;
            }
#pragma unroll
            for (int r = 0; r < RT; ++r)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[r][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[r], af[i], acc[r][i], 0, 0, 0);
        }
    }
    // acc[r][i][e]: output column nb + wn * 16 RT + r * 16 + 4 * (lane / 16) + e of the tile's row wm * 64 + i * 16 + lane % 16
    const bool vec_out = g.ldo % 4 == 0 && g.o_group_stride % 4 == 0 && ((uintptr_t)g.out % 16) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r_in_tile = wm * 64 + i * 16 + l16;
        if (r_in_tile >= rows) continue;
        const int p = g.perm ? g.perm[row0 + r_in_tile] : row0 + r_in_tile;
        const long long orow = (long long)p * g.ldo + (long long)group * g.o_group_stride;
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const int n = nb + wn * 16 * RT + r * 16 + lq * 4;
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                v[e] = acc[r][i][e];
                if (g.act == GM_ACT_RELU2) { v[e] = fmaxf(v[e], 0.f); v[e] *= v[e]; }
            }
            if (vec_out && n + 3 < g.N) {
                if (g.out_bf16) {
                    uint2 w2;
                    w2.x = pack_bf16x2(v[0], v[1]);
                    w2.y = pack_bf16x2(v[2], v[3]);
                    *reinterpret_cast<uint2*>((bf16_t*)g.out + orow + n) = w2;
                } else {
                    *reinterpret_cast<float4*>((float*)g.out + orow + n) = make_float4(v[0], v[1], v[2], v[3]);
                }
                continue;
            }
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (n + e >= g.N) continue;
                if (g.out_bf16) ((bf16_t*)g.out)[orow + n + e] = f32_to_bf16(v[e]);
                else ((float*)g.out)[orow + n + e] = v[e];
            }
        }
    }
}

// rows_a_tile: 16, 32, 64 or 128 rows of a tile (MT groups of 16); a wave takes 32 weight rows, or 64 where
// the output is wide enough to fill the chip with such waves (`wide`).
static int g_grouped_variant = 0;       // measurements only: 0 = choose; 1 = narrow waves; 2 = wide waves; 3, 4 = through LDS, 128 / 256 weight rows
static int g_grouped_bm = 0;            // measurements only: rows of an experts' tile (0 = choose; 64 or 128)
extern "C" void xr_grouped_set_variant(int v, int bm) { g_grouped_variant = v; g_grouped_bm = (bm == 64 || bm == 128) ? bm : 0; }

static int launch_grouped(const GroupedArgs& g, int n_tiles_max, int rows_a_tile, hipStream_t stream) {
    bool wide = g.N >= 128 && rows_a_tile >= 64 && (long long)n_tiles_max * ((g.N + 255) / 256) >= 256;    // enough such workgroups for the chip
    if (g_grouped_variant == 1) wide = false;
    if (g_grouped_variant == 2) wide = rows_a_tile >= 64;
    if (rows_a_tile == 128 && g.N >= 128 && g_grouped_variant != 1 && g_grouped_variant != 2) {     // operands through LDS
        // (256 weight rows a workgroup, 64 x 128 results a wave, was measured slower: sort, both products and
        // the sum took 176 us against 126 for 4,096 rows over 16 experts of 1,024 x 2,048; it stays for measurements)
        const bool big = g_grouped_variant == 4;
        const int bn = big ? 256 : 128;
        const dim3 grid_lds(n_tiles_max, (g.N + bn - 1) / bn);
        if (big) k_grouped_gemm_lds<8><<<grid_lds, 256, 0, stream>>>(g);
        else k_grouped_gemm_lds<4><<<grid_lds, 256, 0, stream>>>(g);
        return 0;
    }
    const int per_wg = wide ? 256 : 128;                    // 4 waves x 4 or 2 groups of 16 weight rows
    const dim3 grid(n_tiles_max, (g.N + per_wg - 1) / per_wg);
    if (rows_a_tile == 16) k_grouped_gemm<1, 2><<<grid, 256, 0, stream>>>(g);
    else if (rows_a_tile == 32) k_grouped_gemm<2, 2><<<grid, 256, 0, stream>>>(g);
    else if (rows_a_tile == 64 && !wide) k_grouped_gemm<4, 2><<<grid, 256, 0, stream>>>(g);
    else if (rows_a_tile == 64) k_grouped_gemm<4, 4><<<grid, 256, 0, stream>>>(g);
    else if (!wide) k_grouped_gemm<8, 2><<<grid, 256, 0, stream>>>(g);
    else k_grouped_gemm<8, 4><<<grid, 256, 0, stream>>>(g);
    return 0;
}

static bool grouped_operands_ok(const void* a, const void* w, int K, int lda, long long a_gs, long long w_gs) {
    return K % 8 == 0 && lda % 8 == 0 && a_gs % 8 == 0 && w_gs % 8 == 0 && ((uintptr_t)a % 16) == 0 && ((uintptr_t)w % 16) == 0;
}

// out[t][g][:N] = w[g] @ a[t][g][:K] for G groups and T rows; a, out: column ranges of wider rows.
extern "C" int xr_heads_gemm_bf16(void* out, const void* a, const void* w, int T, int G, int N, int K, int lda,
                                  long long a_group_stride, int ldo, long long o_group_stride, int out_dtype, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && G > 0 && N > 0 && K > 0, "heads_gemm: bad sizes T=%d G=%d N=%d K=%d", T, G, N, K);
    XR_REQUIRE(out_dtype == XR_F32 || out_dtype == XR_BF16, "heads_gemm: bad output dtype %d", out_dtype);
    XR_REQUIRE(grouped_operands_ok(a, w, K, lda, a_group_stride, (long long)N * K),
               "heads_gemm: K, the row stride and the groups' offsets must be multiples of 8 and the operands 16-byte aligned");
    if (T == 0) return XR_OK;
    const int bm = T <= 16 ? 16 : (T <= 32 ? 32 : 64);
    GroupedArgs g{};
    g.a = (const bf16_t*)a; g.w = (const bf16_t*)w; g.out = out;
    g.a_group_stride = a_group_stride; g.w_group_stride = (long long)N * K; g.o_group_stride = o_group_stride;
    g.lda = lda; g.ldo = ldo; g.N = N; g.K = K; g.out_bf16 = out_dtype == XR_BF16; g.act = GM_ACT_NONE;
    g.gather_div = 1; g.T = T; g.tiles_per_group = (T + bm - 1) / bm;
    XR_REQUIRE((long long)G * g.tiles_per_group <= 0x7fffffffLL, "heads_gemm: too many tiles");
    launch_grouped(g, G * g.tiles_per_group, bm, stream);
    XR_CHECK_LAUNCH("heads_gemm");
    return XR_OK;
}

// ---------------------------------------------------------------- the experts' rows, sorted by expert
// A = T * top choices idx[a] (a = token * top + j).  One workgroup: counts, offsets, the list `perm` of
// the choices expert by expert (in any order inside an expert: a row's result does not depend on
// its place), and the tiles of `bm` rows: tile_group / tile_start / tile_count, n_tiles[0] of them.
#define SORT_MAX_EXPERTS 1024
__global__ __launch_bounds__(1024) void k_moe_sort(const int* __restrict__ idx, int A, int n, int bm, int* __restrict__ perm,
                                                    int* __restrict__ tile_group, int* __restrict__ tile_start,
                                                    int* __restrict__ tile_count, int* __restrict__ n_tiles) {
    __shared__ int count[SORT_MAX_EXPERTS], offset[SORT_MAX_EXPERTS], cursor[SORT_MAX_EXPERTS];
    for (int e = threadIdx.x; e < n; e += 1024) { count[e] = 0; cursor[e] = 0; }
    __syncthreads();
    for (int a = threadIdx.x; a < A; a += 1024) atomicAdd(&count[min(max(idx[a], 0), n - 1)], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0, t = 0;
        for (int e = 0; e < n; ++e) {
            offset[e] = at;
            for (int s = 0; s < count[e]; s += bm) {
                tile_group[t] = e;
                tile_start[t] = at + s;
                tile_count[t] = count[e] - s < bm ? count[e] - s : bm;
                ++t;
            }
            at += count[e];
        }
        n_tiles[0] = t;
    }
    __syncthreads();
    for (int a = threadIdx.x; a < A; a += 1024) {
        const int e = min(max(idx[a], 0), n - 1);
        perm[offset[e] + atomicAdd(&cursor[e], 1)] = a;
    }
}

// y[t] (+)= sum_j wts[t][j] * yz[t * top + j], in the order of the choice
__global__ void k_moe_combine(float* __restrict__ y, const float* __restrict__ yz, const float* __restrict__ wts, int E, int ld_y,
                              int top, size_t n, int accumulate) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / E;
    const int c = (int)(i - t * E);
    float s = 0.f;
    for (int j = 0; j < top; ++j) s += wts[t * top + j] * yz[(t * top + j) * E + c];
    float* o = y + t * ld_y + c;
    *o = accumulate ? *o + s : s;
}

// The routed experts over many rows: sort, z = relu(up)^2 by expert, yz = down by expert, y = the weighted sum.
// scratch: ints [A + 3 * (ceil(A / 16) + n) + 1]; z: bf16 [A, F]; yz: float [A, E].
// Gated experts (`gu` given: float [A, 2F]; w_up [n, 2F, E], an expert's gate rows before its up rows): the first
// product leaves both branches in 32 bits and the gate's own kernel makes z = silu(gate) * up of them.
extern "C" int xr_gate_mul(void* out, const void* gu, int T, int F, int ld_gu, int dtype, int out_dtype, int act, float param,
                           hipStream_t stream);
extern "C" int xr_moe_experts_grouped(float* y, void* z, float* yz, int* scratch, const void* h, const void* w_up,
                                      const void* w_down, const int* idx, const float* wts, int T, int E, int F, int ld_h,
                                      int ld_y, int n, int top, int accumulate, float* gu, hipStream_t stream) {
    XR_REQUIRE(T >= 0 && E > 0 && F > 0 && ld_h >= E && ld_y >= E, "moe_experts_grouped: bad sizes T=%d E=%d F=%d", T, E, F);
    XR_REQUIRE(n >= 1 && n <= SORT_MAX_EXPERTS && top >= 1 && top <= n, "moe_experts_grouped: %d experts (at most %d), %d chosen", n,
               SORT_MAX_EXPERTS, top);
    XR_REQUIRE((long long)T * top <= (1 << 24), "moe_experts_grouped: too many rows");
    const int Fu = gu ? 2 * F : F;          // rows of an expert's first matrix
    XR_REQUIRE(grouped_operands_ok(h, w_up, E, ld_h, 0, (long long)Fu * E) && grouped_operands_ok(z, w_down, F, F, 0, (long long)E * F),
               "moe_experts_grouped: widths and row strides must be multiples of 8 and the operands 16-byte aligned");
    if (T == 0) return XR_OK;
    const int A = T * top, avg = A / n;
    // rows of a tile: what an expert has on average, so that few rows do not idle most of a tile's lanes and the
    // experts' weights are streamed by many workgroups; 128 where an expert has that many
    const int bm = g_grouped_bm ? g_grouped_bm : (avg <= 16 ? 16 : avg <= 32 ? 32 : avg < 128 ? 64 : 128);
    const int max_tiles = (A + bm - 1) / bm + n;           // (at most ceil(A / 16) + n, which is what `scratch` has room for)
    int* perm = scratch;
    int* tile_group = perm + A;
    int* tile_start = tile_group + max_tiles;
    int* tile_count = tile_start + max_tiles;
    int* n_tiles = tile_count + max_tiles;
    k_moe_sort<<<1, 1024, 0, stream>>>(idx, A, n, bm, perm, tile_group, tile_start, tile_count, n_tiles);
    GroupedArgs g{};
    g.perm = perm; g.tile_group = tile_group; g.tile_start = tile_start; g.tile_count = tile_count; g.n_tiles = n_tiles;
    g.a_group_stride = 0; g.o_group_stride = 0;
    // up: rows of h by token, results by choice
    g.a = (const bf16_t*)h; g.lda = ld_h; g.w = (const bf16_t*)w_up; g.w_group_stride = (long long)Fu * E;
    g.out = gu ? (void*)gu : z; g.ldo = Fu;
    g.N = Fu; g.K = E; g.out_bf16 = gu ? 0 : 1; g.act = gu ? GM_ACT_NONE : GM_ACT_RELU2; g.gather_div = top;
    launch_grouped(g, max_tiles, bm, stream);
    if (gu) {
        const int rc = xr_gate_mul(z, gu, A, F, 2 * F, XR_F32, XR_BF16, XR_ACT_SILU, 0.f, stream);
        if (rc != XR_OK) return rc;
    }
    // down: rows of z by choice, results by choice
    g.a = (const bf16_t*)z; g.lda = F; g.w = (const bf16_t*)w_down; g.w_group_stride = (long long)E * F; g.out = yz; g.ldo = E;
    g.N = E; g.K = F; g.out_bf16 = 0; g.act = GM_ACT_NONE; g.gather_div = 1;
    launch_grouped(g, max_tiles, bm, stream);
    const size_t cnt = (size_t)T * E;
    k_moe_combine<<<(unsigned)((cnt + 255) / 256), 256, 0, stream>>>(y, yz, wts, E, ld_y, top, cnt, accumulate);
    XR_CHECK_LAUNCH("moe_experts_grouped");
    return XR_OK;
}
