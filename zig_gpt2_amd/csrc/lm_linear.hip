// lm_linear.hip — the linear maps of the layered-model tier: C = act(A B^T) with fp32 activation rows A and bf16 weights B.
//
// Two kernels behind one launcher:
//   * lm_gemv_kernel   up to 8 rows (decode steps): a wave owns two weight rows, its lanes split K in 16-byte pieces, the
//                      activation rows come straight from the cache hierarchy, sums are fp32 FMAs in both precision modes.
//   * lm_gemm_kernel   prompt portions: 64 x 64 or 128 x 128 tiles on the matrix cores, four waves in a 2 x 2 arrangement of
//                      32 x 32 MFMA tiles.  bf16 mode rounds the activations to bf16 on their way into the LDS and multiplies with
//                      v_mfma_f32_32x32x16_bf16 (fp32 accumulation); 32-bit mode widens the weights and multiplies with
//                      v_mfma_f32_32x32x2_f32.  Any M, N, K: tiles are zero-filled at the edges.
// Both understand the same addressing: a row gather for A, one matrix per grid.z batch (heads), a matrix chosen per batch by
// an index array (the expert of an assignment), and row groups sorted by expert with their offsets in device memory.
#include <stdlib.h>

#include <algorithm>

#include <type_traits>

#include "lm_kernels.h"

namespace zg {
namespace lm {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

struct LinArgs {
    const float* A;
    const bf16_t* B;
    float* C;
    const int* a_rows;
    const int* z_group;
    const int* grp_off;
    long long a_zoff, b_zoff, c_zoff;
    int lda, ldb, ldc;
    int M, N, K;
    int a_div, act, n_groups, a_glu;
    float act_a, act_b;
    int glu_kind;
    float glu_limit;
    const float* glu_scale;
    int glu_gate_col;
    int a_vec, b_vec;  // 16-byte loads allowed (alignment of base, leading dimension and batch offsets)
};

__device__ __forceinline__ float apply_act(float v, const LinArgs& p) {
    const int act = p.act;
    if (act == ACT_SCALE_SOFTCAP) {
        v *= p.act_a;
        if (p.act_b > 0.0f) v = p.act_b * tanhf(v / p.act_b);
    } else if (act == ACT_RELU2) {
        v = fmaxf(v, 0.0f);
        v = v * v;
    } else if (act == ACT_GELU_ERF) {
        v = 0.5f * v * (1.0f + erff(v * 0.70710678118654752f));
    }
    return v;
}

// the gated activation of a [gate | up] row, applied where a product reads it (sc: the row's factor, clipped form only)
__device__ __forceinline__ float glu_on_load(float g, float u, const LinArgs& p, float sc) {
    if (p.glu_kind == GLU_CLIPPED) {
        g = fminf(g * sc, p.glu_limit);
        u = fminf(fmaxf(u * sc, -p.glu_limit), p.glu_limit);
        return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
    }
    return g / (1.0f + expf(-g)) * u;
}

// eight consecutive weights of row `w` from column k, zero beyond K
__device__ __forceinline__ void load_w8(const bf16_t* w, int k, int K, bool vec, float out[8]) {
    if (vec && k + 8 <= K) {
        const u32x4 p = *reinterpret_cast<const u32x4*>(w + k);
        out[0] = bf16_lo(p.x); out[1] = bf16_hi(p.x); out[2] = bf16_lo(p.y); out[3] = bf16_hi(p.y);
        out[4] = bf16_lo(p.z); out[5] = bf16_hi(p.z); out[6] = bf16_lo(p.w); out[7] = bf16_hi(p.w);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) out[i] = (k + i < K) ? __uint_as_float((uint32_t)w[k + i] << 16) : 0.0f;
    }
}

__device__ __forceinline__ f32x4 load_a4(const float* a, int k, int K, bool vec) {
    if (a == nullptr) return f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    if (vec && k + 4 <= K) return *reinterpret_cast<const f32x4*>(a + k);
    f32x4 r;
    r.x = (k + 0 < K) ? a[k + 0] : 0.0f;
    r.y = (k + 1 < K) ? a[k + 1] : 0.0f;
    r.z = (k + 2 < K) ? a[k + 2] : 0.0f;
    r.w = (k + 3 < K) ? a[k + 3] : 0.0f;
    return r;
}

// ------------------------------------------------------------------------------------------------ few rows
template <int MR>
__device__ __forceinline__ void gemv_body(const LinArgs& p, const int z) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 8 + wave * 2;
    if (n0 >= p.N) return;
    const bf16_t* B = p.B + (long long)(p.z_group ? p.z_group[z] : z) * p.b_zoff;
    const float* A = p.A + (long long)z * p.a_zoff;
    float* C = p.C + (long long)z * p.c_zoff;
    const float* arow[MR];
    float asc[MR], agate[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        arow[m] = nullptr;
        asc[m] = agate[m] = 1.0f;
        if (m < p.M) {
            const int rid = p.z_group ? z * p.M + m : m;
            const int src = (p.a_rows ? p.a_rows[rid] : rid) / p.a_div;
            arow[m] = A + (long long)src * p.lda;
            if (p.a_glu > 0 && p.glu_scale) asc[m] = p.glu_scale[rid];
            if (p.a_glu > 0 && p.glu_gate_col >= 0) agate[m] = 1.0f / (1.0f + expf(-arow[m][p.glu_gate_col]));
        }
    }
    const bool two = n0 + 1 < p.N;
    const bf16_t* w0 = B + (long long)n0 * p.ldb;
    const bf16_t* w1 = B + (long long)(two ? n0 + 1 : n0) * p.ldb;
    float acc0[MR], acc1[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc0[m] = acc1[m] = 0.0f;
    // two K pieces per trip, all four weight vectors requested before the first is used: rows of up to 1024 columns cost one
    // memory round trip
    constexpr int U = MR <= 2 ? 2 : 1;
    for (int k = lane * 8; k < p.K; k += 512 * U) {
        float wa[U][8], wb[U][8];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            load_w8(w0, k + 512 * u, p.K, p.b_vec, wa[u]);
            load_w8(w1, k + 512 * u, p.K, p.b_vec, wb[u]);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            f32x4 av[U][2];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kk = k + 512 * u;
                f32x4 a0 = load_a4(arow[m], kk, p.K, p.a_vec), a1 = load_a4(arow[m], kk + 4, p.K, p.a_vec);
                if (p.a_glu > 0 && arow[m]) {  // rows [gate | up]: silu(gate) * up
                    const f32x4 u0 = load_a4(arow[m] + p.a_glu, kk, p.K, p.a_vec && p.a_glu % 4 == 0);
                    const f32x4 u1 = load_a4(arow[m] + p.a_glu, kk + 4, p.K, p.a_vec && p.a_glu % 4 == 0);
                    a0.x = glu_on_load(a0.x, u0.x, p, asc[m]) * agate[m]; a0.y = glu_on_load(a0.y, u0.y, p, asc[m]) * agate[m];
                    a0.z = glu_on_load(a0.z, u0.z, p, asc[m]) * agate[m]; a0.w = glu_on_load(a0.w, u0.w, p, asc[m]) * agate[m];
                    a1.x = glu_on_load(a1.x, u1.x, p, asc[m]) * agate[m]; a1.y = glu_on_load(a1.y, u1.y, p, asc[m]) * agate[m];
                    a1.z = glu_on_load(a1.z, u1.z, p, asc[m]) * agate[m]; a1.w = glu_on_load(a1.w, u1.w, p, asc[m]) * agate[m];
                }
                av[u][0] = a0;
                av[u][1] = a1;
            }
            float s0 = acc0[m], s1 = acc1[m];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const f32x4 a0 = av[u][0], a1 = av[u][1];
                s0 = fmaf(a0.x, wa[u][0], s0); s1 = fmaf(a0.x, wb[u][0], s1);
                s0 = fmaf(a0.y, wa[u][1], s0); s1 = fmaf(a0.y, wb[u][1], s1);
                s0 = fmaf(a0.z, wa[u][2], s0); s1 = fmaf(a0.z, wb[u][2], s1);
                s0 = fmaf(a0.w, wa[u][3], s0); s1 = fmaf(a0.w, wb[u][3], s1);
                s0 = fmaf(a1.x, wa[u][4], s0); s1 = fmaf(a1.x, wb[u][4], s1);
                s0 = fmaf(a1.y, wa[u][5], s0); s1 = fmaf(a1.y, wb[u][5], s1);
                s0 = fmaf(a1.z, wa[u][6], s0); s1 = fmaf(a1.z, wb[u][6], s1);
                s0 = fmaf(a1.w, wa[u][7], s0); s1 = fmaf(a1.w, wb[u][7], s1);
            }
            acc0[m] = s0;
            acc1[m] = s1;
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        const float s0 = wave_allsum(acc0[m]), s1 = wave_allsum(acc1[m]);
        if (lane == 0 && m < p.M) {
            C[(long long)m * p.ldc + n0] = apply_act(s0, p);
            if (two) C[(long long)m * p.ldc + n0 + 1] = apply_act(s1, p);
        }
    }
}

template <int MR>
__global__ __launch_bounds__(256) void lm_gemv_kernel(const LinArgs p) {
    gemv_body<MR>(p, blockIdx.z);
}

// Two products of one-row batches in one launch: batches [0, nz_a) are product a's, the rest product b's (the chosen experts and the
// expert every token uses read the same rows; a decode step saves a dependent launch per product).
__global__ __launch_bounds__(256) void lm_gemv_pair_kernel(const LinArgs a, const LinArgs b, int nz_a) {
    if ((int)blockIdx.z < nz_a) gemv_body<1>(a, blockIdx.z);
    else gemv_body<1>(b, blockIdx.z - nz_a);
}

// The same for long rows (K >= 1536; at 1024 columns half the lanes of a quarter idle and it measured 6 % slower): a workgroup owns two weight rows and its four waves split K into quarters, so a matrix of
// a few MB is requested whole in one go by thousands of waves instead of trip by trip by a few hundred (a 1600 x 1600 matrix:
// 800 workgroups, every 16-byte piece in flight at once); the quarter sums meet in the LDS.  The summation order of an output
// depends on K alone.
template <int MR>
__global__ __launch_bounds__(256) void lm_gemv_ks_kernel(const LinArgs p) {
    __shared__ float s_part[4][MR][2];
    const int z = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * 2;
    const bf16_t* B = p.B + (long long)(p.z_group ? p.z_group[z] : z) * p.b_zoff;
    const float* A = p.A + (long long)z * p.a_zoff;
    float* C = p.C + (long long)z * p.c_zoff;
    const float* arow[MR];
    float asc[MR], agate[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        arow[m] = nullptr;
        asc[m] = agate[m] = 1.0f;
        if (m < p.M) {
            const int rid = p.z_group ? z * p.M + m : m;
            const int src = (p.a_rows ? p.a_rows[rid] : rid) / p.a_div;
            arow[m] = A + (long long)src * p.lda;
            if (p.a_glu > 0 && p.glu_scale) asc[m] = p.glu_scale[rid];
            if (p.a_glu > 0 && p.glu_gate_col >= 0) agate[m] = 1.0f / (1.0f + expf(-arow[m][p.glu_gate_col]));
        }
    }
    const bf16_t* w0 = B + (long long)n0 * p.ldb;
    const bf16_t* w1 = B + (long long)min(n0 + 1, p.N - 1) * p.ldb;
    float acc0[MR], acc1[MR];
#pragma unroll
    for (int m = 0; m < MR; ++m) acc0[m] = acc1[m] = 0.0f;
    const int kq = (((p.K + 3) / 4) + 7) & ~7;  // a wave's quarter of K, a multiple of 8
    const int k_lo = wave * kq, k_hi = min(p.K, k_lo + kq);
    constexpr int U = 2;
    for (int k = k_lo + lane * 8; k < k_hi; k += 512 * U) {
        float wa[U][8], wb[U][8];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            load_w8(w0, k + 512 * u, k_hi, p.b_vec, wa[u]);
            load_w8(w1, k + 512 * u, k_hi, p.b_vec, wb[u]);
        }
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            float s0 = acc0[m], s1 = acc1[m];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int kk = k + 512 * u;
                f32x4 a0 = load_a4(arow[m], kk, k_hi, p.a_vec), a1 = load_a4(arow[m], kk + 4, k_hi, p.a_vec);
                if (p.a_glu > 0 && arow[m]) {  // rows [gate | up]: silu(gate) * up
                    const f32x4 u0 = load_a4(arow[m] + p.a_glu, kk, k_hi, p.a_vec && p.a_glu % 4 == 0);
                    const f32x4 u1 = load_a4(arow[m] + p.a_glu, kk + 4, k_hi, p.a_vec && p.a_glu % 4 == 0);
                    a0.x = glu_on_load(a0.x, u0.x, p, asc[m]) * agate[m]; a0.y = glu_on_load(a0.y, u0.y, p, asc[m]) * agate[m];
                    a0.z = glu_on_load(a0.z, u0.z, p, asc[m]) * agate[m]; a0.w = glu_on_load(a0.w, u0.w, p, asc[m]) * agate[m];
                    a1.x = glu_on_load(a1.x, u1.x, p, asc[m]) * agate[m]; a1.y = glu_on_load(a1.y, u1.y, p, asc[m]) * agate[m];
                    a1.z = glu_on_load(a1.z, u1.z, p, asc[m]) * agate[m]; a1.w = glu_on_load(a1.w, u1.w, p, asc[m]) * agate[m];
                }
                s0 = fmaf(a0.x, wa[u][0], s0); s1 = fmaf(a0.x, wb[u][0], s1);
                s0 = fmaf(a0.y, wa[u][1], s0); s1 = fmaf(a0.y, wb[u][1], s1);
                s0 = fmaf(a0.z, wa[u][2], s0); s1 = fmaf(a0.z, wb[u][2], s1);
                s0 = fmaf(a0.w, wa[u][3], s0); s1 = fmaf(a0.w, wb[u][3], s1);
                s0 = fmaf(a1.x, wa[u][4], s0); s1 = fmaf(a1.x, wb[u][4], s1);
                s0 = fmaf(a1.y, wa[u][5], s0); s1 = fmaf(a1.y, wb[u][5], s1);
                s0 = fmaf(a1.z, wa[u][6], s0); s1 = fmaf(a1.z, wb[u][6], s1);
                s0 = fmaf(a1.w, wa[u][7], s0); s1 = fmaf(a1.w, wb[u][7], s1);
            }
            acc0[m] = s0;
            acc1[m] = s1;
        }
    }
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        const float t0 = wave_allsum(acc0[m]), t1 = wave_allsum(acc1[m]);
        if (lane == 0) {
            s_part[wave][m][0] = t0;
            s_part[wave][m][1] = t1;
        }
    }
    __syncthreads();
    if (threadIdx.x < MR * 2) {
        const int m = threadIdx.x >> 1, c = threadIdx.x & 1;
        if (m < p.M && n0 + c < p.N)
            C[(long long)m * p.ldc + n0 + c] = apply_act((s_part[0][m][c] + s_part[1][m][c]) + (s_part[2][m][c] + s_part[3][m][c]), p);
    }
}

// ------------------------------------------------------------------------------------------------ matrix cores
template <bool F32>
struct Tile {
    static constexpr int BK = F32 ? 16 : 32;
    static constexpr int LDS_K = F32 ? 17 : 40;  // row stride in elements: conflict-free fragment reads
    typedef typename std::conditional<F32, float, bf16_t>::type elem;
};

template <bool F32, int WT>  // WT x WT MFMA tiles of 32 x 32 per wave; workgroup tile = 64 WT squared
__global__ __launch_bounds__(256) void lm_gemm_kernel(const LinArgs p) {
    typedef Tile<F32> T;
    typedef typename T::elem elem;
    constexpr int BM = 64 * WT, BN = 64 * WT, BK = T::BK, LK = T::LDS_K;
    __shared__ __attribute__((aligned(16))) elem As[BM * LK];
    __shared__ __attribute__((aligned(16))) elem Bs[BN * LK];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wy = wave >> 1, wx = wave & 1;
    const int z = blockIdx.z;
    const bf16_t* B = p.B;
    int m0, m_end;
    if (p.grp_off) {  // find the row group this tile belongs to
        int tile = blockIdx.y, e = 0, lo = 0, hi = 0;
        for (; e < p.n_groups; ++e) {
            lo = p.grp_off[e];
            hi = p.grp_off[e + 1];
            const int nt = (hi - lo + BM - 1) / BM;
            if (tile < nt) break;
            tile -= nt;
        }
        if (e >= p.n_groups) return;
        m0 = lo + tile * BM;
        m_end = hi;
        B += (long long)e * p.b_zoff;
    } else {
        m0 = blockIdx.y * BM;
        m_end = p.M;
        B += (long long)(p.z_group ? p.z_group[z] : z) * p.b_zoff;
    }
    const float* A = p.A + (long long)z * p.a_zoff;
    float* C = p.C + (long long)z * p.c_zoff;
    const int n0 = blockIdx.x * BN;

    // global -> register assignment of this thread (fixed over the K loop)
    constexpr int A_VEC_PER_ROW = BK / 4;                 // float4 per A row of the tile
    constexpr int A_LOADS = BM * A_VEC_PER_ROW / 256;     // per thread
    constexpr int B_VEC_PER_ROW = BK / 8;                 // 8 bf16 per vector
    constexpr int B_LOADS = (BN * B_VEC_PER_ROW + 255) / 256;
    const float* a_src[A_LOADS];
    int a_r[A_LOADS], a_k[A_LOADS];
#pragma unroll
    for (int j = 0; j < A_LOADS; ++j) {
        const int v = tid + 256 * j;
        a_r[j] = v / A_VEC_PER_ROW;
        a_k[j] = (v % A_VEC_PER_ROW) * 4;
        const int m = m0 + a_r[j];
        a_src[j] = nullptr;
        if (m < m_end) {
            const int rid = p.z_group ? z * p.M + m : m;
            const int src = (p.a_rows ? p.a_rows[rid] : rid) / p.a_div;
            a_src[j] = A + (long long)src * p.lda;
        }
    }
    const bf16_t* b_src[B_LOADS];
    int b_r[B_LOADS], b_k[B_LOADS];
#pragma unroll
    for (int j = 0; j < B_LOADS; ++j) {
        const int v = tid + 256 * j;
        b_r[j] = v / B_VEC_PER_ROW;
        b_k[j] = (v % B_VEC_PER_ROW) * 8;
        const int n = n0 + b_r[j];
        b_src[j] = (b_r[j] < BN && n < p.N) ? B + (long long)n * p.ldb : nullptr;
    }

    f32x16 acc[WT][WT];
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    f32x4 a_reg[A_LOADS];
    float b_reg[B_LOADS][8];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) a_reg[j] = load_a4(a_src[j], k0 + a_k[j], p.K, p.a_vec);
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            if (b_src[j]) {
                load_w8(b_src[j], k0 + b_k[j], p.K, p.b_vec, b_reg[j]);
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) b_reg[j][i] = 0.0f;
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int j = 0; j < A_LOADS; ++j) {
            elem* d = &As[a_r[j] * LK + a_k[j]];
            if constexpr (F32) {
                d[0] = a_reg[j].x; d[1] = a_reg[j].y; d[2] = a_reg[j].z; d[3] = a_reg[j].w;
            } else {
                u32x2 pk;
                pk.x = cvt_pk_bf16(a_reg[j].x, a_reg[j].y);
                pk.y = cvt_pk_bf16(a_reg[j].z, a_reg[j].w);
                *reinterpret_cast<u32x2*>(d) = pk;
            }
        }
#pragma unroll
        for (int j = 0; j < B_LOADS; ++j) {
            if (b_r[j] < BN) {
                elem* d = &Bs[b_r[j] * LK + b_k[j]];
                if constexpr (F32) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) d[i] = b_reg[j][i];
                } else {
                    u32x4 pk;  // the values are bf16 already: the conversion is exact
                    pk.x = cvt_pk_bf16(b_reg[j][0], b_reg[j][1]);
                    pk.y = cvt_pk_bf16(b_reg[j][2], b_reg[j][3]);
                    pk.z = cvt_pk_bf16(b_reg[j][4], b_reg[j][5]);
                    pk.w = cvt_pk_bf16(b_reg[j][6], b_reg[j][7]);
                    *reinterpret_cast<u32x4*>(d) = pk;
                }
            }
        }
    };

    fetch(0);
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        __syncthreads();  // the previous step's fragment reads are done
        stash();
        __syncthreads();
        if (k0 + BK < p.K) fetch(k0 + BK);  // in flight beside the MFMAs
        const int r = lane & 31, kh = lane >> 5;
        if constexpr (F32) {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 2) {
                float af[WT], bf[WT];
#pragma unroll
                for (int i = 0; i < WT; ++i) af[i] = As[((wy * WT + i) * 32 + r) * LK + kk + kh];
#pragma unroll
                for (int j = 0; j < WT; ++j) bf[j] = Bs[((wx * WT + j) * 32 + r) * LK + kk + kh];
#pragma unroll
                for (int i = 0; i < WT; ++i)
#pragma unroll
                    for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 16) {
                bf16x8 af[WT], bf[WT];
#pragma unroll
                for (int i = 0; i < WT; ++i)
                    af[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&As[((wy * WT + i) * 32 + r) * LK + kk + kh * 8]));
#pragma unroll
                for (int j = 0; j < WT; ++j)
                    bf[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Bs[((wx * WT + j) * 32 + r) * LK + kk + kh * 8]));
#pragma unroll
                for (int i = 0; i < WT; ++i)
#pragma unroll
                    for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bf[j], acc[i][j], 0, 0, 0);
            }
        }
    }

    // accumulator element e of a 32 x 32 tile: row 8 (e / 4) + 4 (lane / 32) + e % 4, column lane % 32
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) {
            const int n = n0 + (wx * WT + j) * 32 + (lane & 31);
            if (n >= p.N) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int m = m0 + (wy * WT + i) * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (m < m_end) C[(long long)m * p.ldc + n] = apply_act(acc[i][j][e], p);
            }
        }
}

}  // namespace

namespace {
LinArgs make_args(const Linear& L);
bool takes_k_split(const Linear& L) { return L.K >= 1536 && L.M <= 2 && L.nz <= 4; }
}  // namespace

int launch_linear_pair(const Linear& A, const Linear& B, bool f32, hipStream_t s) {
    const bool one_launch = A.M == 1 && B.M == 1 && A.nz >= 1 && B.nz >= 1 && A.N > 0 && B.N > 0 && !A.grp_off && !B.grp_off && !takes_k_split(A) &&
                            !takes_k_split(B) && A.K > 0 && B.K > 0 && A.A && A.B && A.C && B.A && B.B && B.C && A.a_div >= 1 && B.a_div >= 1 &&
                            A.nz + B.nz <= 65535;
    if (!one_launch) {
        ZG_TRY(launch_linear(A, f32, s));
        return launch_linear(B, f32, s);
    }
    const dim3 grid((std::max(A.N, B.N) + 7) / 8, 1, A.nz + B.nz);
    lm_gemv_pair_kernel<<<grid, 256, 0, s>>>(make_args(A), make_args(B), A.nz);
    note_kernel("lm_gemv_pair_kernel");
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

namespace {
LinArgs make_args(const Linear& L) {
    LinArgs p;
    p.A = L.A; p.B = L.B; p.C = L.C; p.a_rows = L.a_rows; p.z_group = L.z_group; p.grp_off = L.grp_off;
    p.a_zoff = L.a_zoff; p.b_zoff = L.b_zoff; p.c_zoff = L.c_zoff;
    p.lda = L.lda; p.ldb = L.ldb; p.ldc = L.ldc; p.M = L.M; p.N = L.N; p.K = L.K;
    p.a_div = L.a_div; p.act = L.act; p.n_groups = L.grp_off ? L.n_groups : 0; p.a_glu = L.a_glu;
    p.act_a = L.act_a; p.act_b = L.act_b; p.glu_kind = L.glu_kind; p.glu_limit = L.glu_limit; p.glu_scale = L.glu_scale;
    p.glu_gate_col = L.glu_gate_col;
    p.a_vec = ((reinterpret_cast<uintptr_t>(L.A) & 15) == 0 && L.lda % 4 == 0 && L.a_zoff % 4 == 0) ? 1 : 0;
    p.b_vec = ((reinterpret_cast<uintptr_t>(L.B) & 15) == 0 && L.ldb % 8 == 0 && L.b_zoff % 8 == 0) ? 1 : 0;
    return p;
}
}  // namespace

int launch_linear(const Linear& L, bool f32, hipStream_t s) {
    if (L.M <= 0 || L.N <= 0 || L.nz <= 0) return ZG_OK;
    ZG_REQUIRE(L.K > 0 && L.A && L.B && L.C, ZG_ERR_ARG, "linear: empty operand");
    ZG_REQUIRE(L.a_div >= 1, ZG_ERR_ARG, "linear: a_div %d", L.a_div);
    const LinArgs p = make_args(L);
    if (!L.grp_off && L.M <= kGemvMaxRows) {
        if (takes_k_split(L)) {  // long rows, one or two of them, few batches: K split over the waves, two weight rows per workgroup
            const dim3 gks((L.N + 1) / 2, 1, L.nz);  // (from four rows on the activations are re-read by too many workgroups: measured slower)
            if (L.M == 1) lm_gemv_ks_kernel<1><<<gks, 256, 0, s>>>(p);
            else lm_gemv_ks_kernel<2><<<gks, 256, 0, s>>>(p);
            note_kernel("lm_gemv_ks_kernel<%d>", L.M);
            ZG_HIP(hipGetLastError());
            return ZG_OK;
        }
        const dim3 grid((L.N + 7) / 8, 1, L.nz);
        if (L.M == 1) lm_gemv_kernel<1><<<grid, 256, 0, s>>>(p);
        else if (L.M == 2) lm_gemv_kernel<2><<<grid, 256, 0, s>>>(p);
        else if (L.M <= 4) lm_gemv_kernel<4><<<grid, 256, 0, s>>>(p);
        else lm_gemv_kernel<8><<<grid, 256, 0, s>>>(p);
        note_kernel("lm_gemv_kernel<%d>", L.M == 1 ? 1 : L.M == 2 ? 2 : L.M <= 4 ? 4 : 8);
        ZG_HIP(hipGetLastError());
        return ZG_OK;
    }
    ZG_REQUIRE(L.a_glu == 0, ZG_ERR_ARG, "linear: the gated activation on load is for steps of few rows");
    ZG_REQUIRE(!(L.z_group && L.grp_off), ZG_ERR_ARG, "linear: a matrix per batch and row groups exclude each other");
    // 64 x 64 tiles.  The 128 x 128 form of the same kernel measured slower at every size tried (a prompt pass of 8 x 1023
    // tokens at width 1600: 143 against 127 ms; width 768: 14.6 against 12.9 ms) and is kept behind ZGPT2_LM_GEMM_TILE=128 only
    // (tests run ragged shapes through it).
    bool big = false;
    if (const char* e = getenv("ZGPT2_LM_GEMM_TILE")) big = atoi(e) == 128;
    const int b = big ? 128 : 64;
    const dim3 grid((L.N + b - 1) / b, (L.M + b - 1) / b + (L.grp_off ? L.n_groups : 0), L.nz);
    ZG_REQUIRE(grid.y <= 65535 && grid.z <= 65535, ZG_ERR_UNSUPPORTED, "linear: %d rows in %d batches exceed the grid", L.M, L.nz);
    if (f32) {
        if (big) lm_gemm_kernel<true, 2><<<grid, 256, 0, s>>>(p);
        else lm_gemm_kernel<true, 1><<<grid, 256, 0, s>>>(p);
    } else {
        if (big) lm_gemm_kernel<false, 2><<<grid, 256, 0, s>>>(p);
        else lm_gemm_kernel<false, 1><<<grid, 256, 0, s>>>(p);
    }
    note_kernel("lm_gemm_kernel<%s, %d>", f32 ? "true" : "false", big ? 2 : 1);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

}  // namespace lm
}  // namespace zg
