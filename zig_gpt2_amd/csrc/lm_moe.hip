// lm_moe.hip — routing of the mixture-of-experts feed-forward of the layered-model tier: router scores and the choice of experts
// (fp32), the sort of a step's assignments by expert for the grouped matrix products, the gated activation, and the weighted
// sum of the chosen experts' outputs fused with the norm and the residual sum behind the sublayer.
#include <math.h>

#include "lm_kernels.h"

namespace zg {
namespace lm {

namespace {

constexpr int kMaxExperts = 256;  // four per lane of the routing wave

__device__ __forceinline__ float block_allsum(float v, float* s_red) {
    v = wave_allsum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) s_red[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nw; ++w) t += s_red[w];
    return t;
}

// One workgroup per row.  The four waves share the experts (wave w scores experts w, w + 4, ...): a router row is one dot
// product, the lanes take 16-byte pieces of it and every piece of up to 2048 channels is requested before the first is used; the
// logits meet in the LDS and wave 0 does the softmax and the choice, lane e % 64 holding expert e (four slots per lane).
// top_logits: the correction is a bias of the logits, the largest logits are chosen and the weights are the softmax over the chosen
// logits alone.
// sigmoid scores with groups: experts ranked by r = sigmoid(z) + correction; a block of adjacent experts ranks by its best r plus
// its second-best r, only the `keep` top-ranked blocks (lowest index wins a tie) remain eligible; the weights are the winners'
// sigmoid(z) over their sum, times out_scale.
// pre.x != null: the workgroup first finishes its own row — x += mult * nb(sum of the sublayer's parts), h = nn(x), both written
// out, h also kept in the LDS — and routes on that (steps of few rows: the sum and norm in front of the router need no launch
// of their own).
__global__ __launch_bounds__(256) void route_kernel(const float* g, int M, int W, const bf16_t* router, const float* correction, int E, int top,
                                                    int* pick, float* weight, int rule, int groups, int keep, float out_scale, const RoutePre pre) {
    const bool top_logits = rule == 1 || rule == 2;  // rules that choose by the logits themselves
    const bool sigmoid_w = rule == 2;   // ... and weigh a chosen expert by sigmoid(z), nothing renormalised
    extern __shared__ __attribute__((aligned(16))) float s_row[];  // [W] with pre
    __shared__ float s_z[kMaxExperts];
    __shared__ float s_gs[kMaxExperts];
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* row = g + (size_t)m * W;
    if (pre.x) {
        const float ab = pre.nb[2 * W], an = pre.nn[2 * W];
        for (int i = threadIdx.x; i < W; i += blockDim.x) {
            const size_t idx = (size_t)m * W + i;
            float a = pre.y.a ? pre.y.a[idx] : 0.0f;
            for (int k = 0; k < pre.y.top; ++k) {
                const size_t as = (size_t)m * pre.y.top + k;
                a = fmaf(pre.y.exp_w ? pre.y.exp_w[as] : 1.0f, pre.y.exp[(size_t)(pre.y.inv ? pre.y.inv[as] : as) * W + i], a);
            }
            if (pre.y.b) a += pre.y.b[idx];
            const float v = fmaf(pre.mult, fmaf(tanhf(ab * a), pre.nb[i], pre.nb[W + i]), pre.x[idx]);
            const float hv = fmaf(tanhf(an * v), pre.nn[i], pre.nn[W + i]);
            pre.x[idx] = v;
            pre.h[idx] = hv;
            s_row[i] = hv;
        }
        __syncthreads();
        row = s_row;
    }
    const bool vec = (W % 8 == 0) && (pre.x || (reinterpret_cast<uintptr_t>(g) & 15) == 0) && ((reinterpret_cast<uintptr_t>(router) & 15) == 0);
    for (int e = wave; e < E; e += 4) {
        const bf16_t* wr = router + (size_t)e * W;
        float a = 0.0f;
        if (vec) {
            for (int k0 = lane * 8; k0 < W; k0 += 2048) {
                f32x4 x0[4], x1[4];
                u32x4 wv[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int k = k0 + 512 * u;
                    const bool ok = k < W;
                    x0[u] = ok ? *reinterpret_cast<const f32x4*>(row + k) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    x1[u] = ok ? *reinterpret_cast<const f32x4*>(row + k + 4) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    wv[u] = ok ? *reinterpret_cast<const u32x4*>(wr + k) : u32x4{0u, 0u, 0u, 0u};
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    a = fmaf(x0[u].x, bf16_lo(wv[u].x), a);
                    a = fmaf(x0[u].y, bf16_hi(wv[u].x), a);
                    a = fmaf(x0[u].z, bf16_lo(wv[u].y), a);
                    a = fmaf(x0[u].w, bf16_hi(wv[u].y), a);
                    a = fmaf(x1[u].x, bf16_lo(wv[u].z), a);
                    a = fmaf(x1[u].y, bf16_hi(wv[u].z), a);
                    a = fmaf(x1[u].z, bf16_lo(wv[u].w), a);
                    a = fmaf(x1[u].w, bf16_hi(wv[u].w), a);
                }
            }
        } else {
            for (int k = lane; k < W; k += 64) a = fmaf(row[k], __uint_as_float((uint32_t)wr[k] << 16), a);
        }
        a = wave_allsum(a);
        if (lane == 0) s_z[e] = a;
    }
    __syncthreads();
    if (rule == 3 && groups > 1) {  // every block's rank, by all four waves: its best r plus its second-best r
        __shared__ float s_c[kMaxExperts];
        const int gsz = E / groups;
        for (int e = threadIdx.x; e < E; e += blockDim.x) s_c[e] = 1.0f / (1.0f + expf(-s_z[e])) + (correction ? correction[e] : 0.0f);
        __syncthreads();
        for (int gi = threadIdx.x; gi < groups; gi += blockDim.x) {
            float a = -INFINITY, b = -INFINITY;
            for (int e = gi * gsz; e < (gi + 1) * gsz; ++e) {
                const float c = s_c[e];
                if (c > a) {
                    b = a;
                    a = c;
                } else if (c > b) {
                    b = c;
                }
            }
            s_gs[gi] = gsz > 1 ? a + b : a;
        }
        __syncthreads();
    }
    if (wave != 0) return;
    float z[4], sc[4], ch[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) z[i] = lane + 64 * i < E ? s_z[lane + 64 * i] : -INFINITY;
    if (top_logits) {
#pragma unroll
        for (int i = 0; i < 4; ++i) ch[i] = lane + 64 * i < E ? z[i] + (correction ? correction[lane + 64 * i] : 0.0f) : -INFINITY;
        float ek[4] = {0.0f, 0.0f, 0.0f, 0.0f};  // exp(z_k - z_0) of choice k on lane k % 64, slot k / 64
        float first = 0.0f;
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY;
            int bi = 0x7fffffff;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (ch[i] > best) {
                    best = ch[i];
                    bi = lane + 64 * i;
                }
            const float wbest = wave_allmax(best);
            int cand = (best == wbest) ? bi : 0x7fffffff;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
            if (cand == 0x7fffffff) cand = 0;
            if (k == 0) first = wbest;
            if ((cand & 63) == lane) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if ((cand >> 6) == i) {
                        pick[(size_t)m * top + k] = cand;
                        if (sigmoid_w) weight[(size_t)m * top + k] = 1.0f / (1.0f + expf(-ch[i]));
                        ch[i] = -INFINITY;
                    }
            }
            if ((k & 63) == lane) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if ((k >> 6) == i) ek[i] = expf(wbest - first);
            }
        }
        if (sigmoid_w) return;
        const float sum = wave_allsum((ek[0] + ek[1]) + (ek[2] + ek[3]));
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (lane + 64 * i < top) weight[(size_t)m * top + lane + 64 * i] = ek[i] / sum;
        return;
    }
    if (rule == 3) {
        int pk[4] = {0, 0, 0, 0};  // 1 + the place of the expert among the chosen
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e = lane + 64 * i;
            sc[i] = e < E ? 1.0f / (1.0f + expf(-z[i])) : 0.0f;
            ch[i] = e < E ? sc[i] + (correction ? correction[e] : 0.0f) : -INFINITY;
        }
        if (groups > 1) {
            const int gsz = E / groups;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int e = lane + 64 * i;
                if (e >= E) continue;
                const int mine = e / gsz;
                const float ms = s_gs[mine];
                int ahead = 0;  // groups that come before this expert's group
                for (int o = 0; o < groups; ++o) ahead += (s_gs[o] > ms || (s_gs[o] == ms && o < mine)) ? 1 : 0;
                if (ahead >= keep) ch[i] = -INFINITY;
            }
        }
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY;
            int bi = 0x7fffffff;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (ch[i] > best) {  // ascending expert index per lane: the first maximum stays
                    best = ch[i];
                    bi = lane + 64 * i;
                }
            const float wbest = wave_allmax(best);
            int cand = (best == wbest) ? bi : 0x7fffffff;
#pragma unroll
            for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
            if (cand == 0x7fffffff) cand = 0;  // nothing left to choose from: keep the indices in range
            if ((cand & 63) == lane) {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if ((cand >> 6) == i) {
                        pick[(size_t)m * top + k] = cand;
                        pk[i] = k + 1;
                        ch[i] = -INFINITY;
                    }
            }
        }
        float mine = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) mine += pk[i] ? sc[i] : 0.0f;
        const float total = wave_allsum(mine) + 1e-20f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (pk[i]) weight[(size_t)m * top + pk[i] - 1] = sc[i] / total * out_scale;
        return;
    }
    const float mx = wave_allmax(fmaxf(fmaxf(z[0], z[1]), fmaxf(z[2], z[3])));
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        sc[i] = expf(z[i] - mx);  // 0 for the experts that do not exist
        sum += sc[i];
    }
    sum = wave_allsum(sum);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int e = lane + 64 * i;
        sc[i] = sc[i] / sum;
        ch[i] = e < E ? sc[i] + correction[e] : -INFINITY;
    }
    for (int k = 0; k < top; ++k) {
        float best = -INFINITY;
        int bi = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            if (ch[i] > best) {  // ascending expert index per lane: the first maximum stays
                best = ch[i];
                bi = lane + 64 * i;
            }
        const float wbest = wave_allmax(best);
        int cand = (best == wbest) ? bi : 0x7fffffff;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
        if (cand == 0x7fffffff) cand = 0;  // nothing left to choose from (NaN scores): keep the indices in range
        if ((cand & 63) == lane) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if ((cand >> 6) == i) {
                    pick[(size_t)m * top + k] = cand;
                    weight[(size_t)m * top + k] = sc[i];
                    ch[i] = -INFINITY;
                }
        }
    }
}

// one workgroup: histogram, offsets, placement.  The order inside a group is arbitrary: every row of a grouped product is
// computed independently of its neighbours, so the results do not depend on it.
__global__ __launch_bounds__(1024) void group_kernel(const int* pick, int n_assign, int E, int* grp_off, int* sorted, int* inv) {
    __shared__ int s_cnt[kMaxExperts], s_off[kMaxExperts + 1], s_cur[kMaxExperts];
    for (int e = threadIdx.x; e < E; e += blockDim.x) s_cnt[e] = s_cur[e] = 0;
    __syncthreads();
    for (int a = threadIdx.x; a < n_assign; a += blockDim.x) atomicAdd(&s_cnt[pick[a]], 1);
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0;
        for (int e = 0; e < E; ++e) {
            s_off[e] = o;
            o += s_cnt[e];
        }
        s_off[E] = o;
    }
    __syncthreads();
    for (int e = threadIdx.x; e <= E; e += blockDim.x) grp_off[e] = s_off[e];
    for (int a = threadIdx.x; a < n_assign; a += blockDim.x) {
        const int e = pick[a];
        const int p = s_off[e] + atomicAdd(&s_cur[e], 1);
        sorted[p] = a;
        inv[a] = p;
    }
}

__global__ __launch_bounds__(256) void glu_kernel(const float* gu, float* h, size_t n, int F) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const size_t r = idx / F;
    const int j = (int)(idx % F);
    const float a = gu[r * 2 * F + j], b = gu[r * 2 * F + F + j];
    h[idx] = a / (1.0f + expf(-a)) * b;
}

// the clipped gated activation: the gate capped from above, the linear part clipped on both sides and lifted by one
__device__ __forceinline__ float glu_clipped_f(float g, float u, float limit) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.0f + expf(-1.702f * g)) * (u + 1.0f);
}

__global__ __launch_bounds__(256) void glu_clipped_kernel(const float* gu, int ld, float* h, size_t n, int F, float limit, const float* row_scale,
                                                          const int* row_of, int gate_col) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const size_t r = idx / F;
    const int j = (int)(idx % F);
    const float* row = gu + r * ld;
    const float sc = row_scale ? row_scale[row_of ? row_of[r] : r] : 1.0f;
    float v = glu_clipped_f(sc * row[j], sc * row[F + j], limit);
    if (gate_col >= 0) v *= 1.0f / (1.0f + expf(-row[gate_col]));
    h[idx] = v;
}

__global__ __launch_bounds__(256) void expert_sum_kernel(float* y, const float* yexp, const int* inv, const float* weight, int top, const float* ys,
                                                         size_t n, int W) {
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const size_t m = idx / W;
    const int i = (int)(idx % W);
    float a = 0.0f;
    for (int k = 0; k < top; ++k) {  // in choice order: the sum does not depend on the batch
        const size_t as = m * top + k;
        const float v = yexp[(size_t)(inv ? inv[as] : as) * W + i];
        a = weight ? fmaf(weight[as], v, a) : a + v;
    }
    if (ys) a += ys[idx];
    y[idx] = a;
}

__global__ __launch_bounds__(256) void moe_combine_kernel(float* x, const float* yexp, const int* inv, const float* weight, int top, const float* w,
                                                          float eps, int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    auto mix = [&](int i) {
        float y = 0.0f;
        for (int k = 0; k < top; ++k) {
            const int a = m * top + k;
            y = fmaf(weight[a], yexp[(size_t)(inv ? inv[a] : a) * W + i], y);
        }
        return y;
    };
    float ss = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float y = mix(i);
        ss = fmaf(y, y, ss);
    }
    ss = block_allsum(ss, s_red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) x[(size_t)m * W + i] += mix(i) * r * (1.0f + w[i]);
}

}  // namespace

int launch_route(const float* g, int M, int W, const bf16_t* router, const float* correction, int E, int top, int* pick, float* weight,
                 int rule, hipStream_t s, int groups, int keep, float out_scale, const RoutePre* pre) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(E >= 1 && E <= kMaxExperts && top >= 1 && top <= E, ZG_ERR_UNSUPPORTED, "router: %d experts, %d chosen (at most %d experts)", E, top,
               kMaxExperts);
    if (groups < 1) groups = 1;
    if (keep < 1) keep = groups;  // (a descriptor that names no groups)
    ZG_REQUIRE(E % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (E / groups), ZG_ERR_ARG,
               "router: %d experts in %d groups, %d groups kept, %d chosen", E, groups, keep, top);
    ZG_REQUIRE(!pre || (pre->x && pre->nb && pre->nn && pre->h == g && W <= kRouteFuseWidth), ZG_ERR_ARG,
               "router: the sum in front of it needs x, both norms, its output as the router's input, and a width of at most %d", kRouteFuseWidth);
    route_kernel<<<M, 256, pre ? (size_t)W * sizeof(float) : 0, s>>>(g, M, W, router, correction, E, top, pick, weight, rule, groups, keep, out_scale,
                                                                     pre ? *pre : RoutePre());
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_group(const int* pick, int n_assign, int E, int* grp_off, int* sorted, int* inv, hipStream_t s) {
    ZG_REQUIRE(E >= 1 && E <= kMaxExperts, ZG_ERR_UNSUPPORTED, "router: %d experts (at most %d)", E, kMaxExperts);
    group_kernel<<<1, 1024, 0, s>>>(pick, n_assign, E, grp_off, sorted, inv);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_glu(const float* gu, float* h, int rows, int F, hipStream_t s) {
    const size_t n = (size_t)rows * F;
    if (n == 0) return ZG_OK;
    glu_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gu, h, n, F);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_glu_clipped(const float* gu, int ld, float* h, int rows, int F, float limit, const float* row_scale, const int* row_of, int gate_col,
                       hipStream_t s) {
    const size_t n = (size_t)rows * F;
    if (n == 0) return ZG_OK;
    glu_clipped_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(gu, ld, h, n, F, limit, row_scale, row_of, gate_col);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_expert_sum(float* y, const float* yexp, const int* inv, const float* weight, int top, const float* ys, int M, int W, hipStream_t s) {
    const size_t n = (size_t)M * W;
    if (n == 0) return ZG_OK;
    expert_sum_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(y, yexp, inv, weight, top, ys, n, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_moe_combine(float* x, const float* yexp, const int* inv, const float* weight, int top, const float* w, float eps, int M, int W,
                       hipStream_t s) {
    if (M <= 0) return ZG_OK;
    moe_combine_kernel<<<M, 256, 0, s>>>(x, yexp, inv, weight, top, w, eps, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

}  // namespace lm
}  // namespace zg
