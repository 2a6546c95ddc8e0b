// lm_mix.hip — the row-wise and sequence-wise kernels of the layered-model tier: embedding, RMS norms (with the token shift and
// the residual sum fused in), the gated linear recurrence (HGRN2) and the latent attention over a paged cache of latents.
// Everything here is fp32 in both precision modes: norms, gates, the recurrent state, positions, angles, scores and weights.
#include <math.h>
#include <stdlib.h>

#include <algorithm>

#include "lm_kernels.h"

namespace zg {
namespace lm {

namespace {

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

// 1 / sqrt(mean(v^2) + eps) of one row, the same summation order wherever a row is normed (a row normed again as somebody's
// predecessor gives the bits its own workgroup got).
__device__ __forceinline__ float row_inv_rms(const float* v, int n, float eps, float* s_red) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss = fmaf(v[i], v[i], ss);
    ss = block_allsum(ss, s_red);
    return 1.0f / sqrtf(ss / (float)n + eps);
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }

__global__ __launch_bounds__(256) void embed_kernel(const bf16_t* table, const int* ids, float* x, float* x_copy, float scale, int W, int vocab,
                                                    int* flag, const int* row_pos, const float* pos_freq) {
    const int m = blockIdx.x, id = ids[m];
    const bool ok = id >= 0 && id < vocab;
    if (!ok && threadIdx.x == 0) *flag = 1;
    const bf16_t* row = table + (size_t)(ok ? id : 0) * W;
    const float fpos = row_pos ? (float)row_pos[m] : 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        float v = ok ? __uint_as_float((uint32_t)row[i] << 16) * scale : 0.0f;
        if (row_pos) {  // entries (2j, 2j + 1) = (sin, cos) of the fp32 product position x frequency j
            const float a = fpos * pos_freq[i >> 1];
            v += (i & 1) ? cosf(a) : sinf(a);
        }
        x[(size_t)m * W + i] = v;
        if (x_copy) x_copy[(size_t)m * W + i] = v;
    }
}

// Rows of up to 256 * kRowRegs floats are held in registers between the statistics and the result: every operand is requested
// in one go at the top of the kernel, so a one-row step (decoding) pays one memory round trip instead of one per pass.
constexpr int kRowRegs = 16;

__global__ __launch_bounds__(256) void norm_shift_kernel(const float* x, const float* w, const float* mu, float eps, float* out, int W,
                                                         const int* row_prev, const int* row_slot, const float* shift_state,
                                                         size_t slot_stride, const int* row_entry_if_last, float* last_out) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* xr = x + (size_t)m * W;
    const int entry = row_entry_if_last ? row_entry_if_last[m] : -1;
    const int pm = mu ? row_prev[m] : -1;
    const float* xp = (mu && pm >= 0) ? x + (size_t)pm * W : nullptr;
    const float* hp = (mu && pm < 0) ? shift_state + (size_t)row_slot[m] * slot_stride : nullptr;
    if (W <= 256 * kRowRegs) {
        float xv[kRowRegs], pv[kRowRegs], wv[kRowRegs], mv[kRowRegs];
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            const bool ok = i < W;
            xv[j] = ok ? xr[i] : 0.0f;
            wv[j] = ok ? w[i] : 0.0f;
            mv[j] = (ok && mu) ? mu[i] : 0.0f;
            pv[j] = !ok ? 0.0f : xp ? xp[i] : hp ? hp[i] : 0.0f;
        }
        float ss = 0.0f;  // the same order as row_inv_rms: element i of thread t is t + 256 j, j ascending
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) ss = fmaf(xv[j], xv[j], ss);
        ss = block_allsum(ss, s_red);
        const float r = 1.0f / sqrtf(ss / (float)W + eps);
        float rp = 0.0f;
        if (xp) {
            float sp = 0.0f;
#pragma unroll
            for (int j = 0; j < kRowRegs; ++j) sp = fmaf(pv[j], pv[j], sp);
            sp = block_allsum(sp, s_red);
            rp = 1.0f / sqrtf(sp / (float)W + eps);
        }
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < W) {
                const float g = 1.0f + wv[j];
                const float h = xv[j] * r * g;
                const float before = xp ? pv[j] * rp * g : pv[j];
                out[(size_t)m * W + i] = mu ? h + (before - h) * mv[j] : h;
                if (entry >= 0) last_out[(size_t)entry * W + i] = h;
            }
        }
        return;
    }
    const float r = row_inv_rms(xr, W, eps, s_red);
    if (mu == nullptr) {
        for (int i = threadIdx.x; i < W; i += blockDim.x) {
            const float h = xr[i] * r * (1.0f + w[i]);
            out[(size_t)m * W + i] = h;
            if (entry >= 0) last_out[(size_t)entry * W + i] = h;
        }
        return;
    }
    float rp = 0.0f;
    if (xp) rp = row_inv_rms(xp, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float g = 1.0f + w[i];
        const float h = xr[i] * r * g;
        const float before = xp ? xp[i] * rp * g : hp[i];
        out[(size_t)m * W + i] = h + (before - h) * mu[i];
        if (entry >= 0) last_out[(size_t)entry * W + i] = h;
    }
}

__global__ __launch_bounds__(256) void commit_rows_kernel(float* dst, size_t slot_stride, const float* src, size_t src_stride, const int* slots,
                                                          int width, size_t dst_set_stride, size_t src_set_stride) {
    const int e = blockIdx.x, set = blockIdx.y;
    float* d = dst + (size_t)slots[e] * slot_stride + set * dst_set_stride;
    const float* s = src + (size_t)e * src_stride + set * src_set_stride;
    for (int i = threadIdx.x; i < width; i += blockDim.x) d[i] = s[i];
}

__global__ __launch_bounds__(256) void norm_add_kernel(float* x, const float* y, const float* w, float eps, int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* yr = y + (size_t)m * W;
    const float r = row_inv_rms(yr, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) x[(size_t)m * W + i] += yr[i] * r * (1.0f + w[i]);
}

// x += norm(y) * (1 + wb), then h = norm(x) * (1 + wn): the norm behind the mixer, the residual sum and the norm in front of the
// feed-forward in one pass over the row
__global__ __launch_bounds__(256) void norm_add_norm_kernel(float* x, const float* y, const float* wb, const float* wn, float eps, float* h, int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* yr = y + (size_t)m * W;
    float* xr = x + (size_t)m * W;
    if (W <= 256 * kRowRegs) {
        float yv[kRowRegs], xv[kRowRegs], bv[kRowRegs], nv[kRowRegs];
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            const bool ok = i < W;
            yv[j] = ok ? yr[i] : 0.0f;
            xv[j] = ok ? xr[i] : 0.0f;
            bv[j] = ok ? wb[i] : 0.0f;
            nv[j] = ok ? wn[i] : 0.0f;
        }
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) ss = fmaf(yv[j], yv[j], ss);
        ss = block_allsum(ss, s_red);
        const float r = 1.0f / sqrtf(ss / (float)W + eps);
        float s2 = 0.0f;
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            xv[j] += yv[j] * r * (1.0f + bv[j]);  // (rows beyond W: 0 + 0)
            s2 = fmaf(xv[j], xv[j], s2);
        }
        s2 = block_allsum(s2, s_red);
        const float r2 = 1.0f / sqrtf(s2 / (float)W + eps);
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < W) {
                xr[i] = xv[j];
                h[(size_t)m * W + i] = xv[j] * r2 * (1.0f + nv[j]);
            }
        }
        return;
    }
    const float r = row_inv_rms(yr, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) xr[i] += yr[i] * r * (1.0f + wb[i]);  // each thread rereads only what it wrote
    float ss = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) ss = fmaf(xr[i], xr[i], ss);
    ss = block_allsum(ss, s_red);
    const float r2 = 1.0f / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) h[(size_t)m * W + i] = xr[i] * r2 * (1.0f + wn[i]);
}

// Steps of one row per entry (decoding): the sum behind a pass's last sublayer and the NEXT pass's norm + token shift in one
// launch, the row held in registers:
//   y = a sublayer's output row, or sum_k weight[k] * yexp[m top + k] (the chosen experts, in choice order)
//   x += norm(y) (1 + wb);   h = norm(x) (1 + wn);   out = h + (state[slot] - h) mu;   last_out[entry] = h
// (the predecessor of a decoded token is always the row its slot keeps)
__global__ __launch_bounds__(256) void sum_norm_shift_kernel(float* x, const float* y, const float* yexp, const float* weight, int top, const float* wb,
                                                             const float* wn, const float* mu, float eps, float* out, int W, const int* row_slot,
                                                             const float* shift_state, size_t slot_stride, const int* row_entry_if_last,
                                                             float* last_out) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    float* xr = x + (size_t)m * W;
    const float* hp = shift_state + (size_t)row_slot[m] * slot_stride;
    const int entry = row_entry_if_last[m];
    float yv[kRowRegs], xv[kRowRegs], bv[kRowRegs], nv[kRowRegs], mv[kRowRegs], pv[kRowRegs];
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
        const int i = threadIdx.x + 256 * j;
        const bool ok = i < W;
        float v = 0.0f;
        if (ok) {
            if (yexp) {
                for (int k = 0; k < top; ++k) v = fmaf(weight[m * top + k], yexp[(size_t)(m * top + k) * W + i], v);
            } else {
                v = y[(size_t)m * W + i];
            }
        }
        yv[j] = v;
        xv[j] = ok ? xr[i] : 0.0f;
        bv[j] = ok ? wb[i] : 0.0f;
        nv[j] = ok ? wn[i] : 0.0f;
        mv[j] = ok ? mu[i] : 0.0f;
        pv[j] = ok ? hp[i] : 0.0f;
    }
    float ss = 0.0f;
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) ss = fmaf(yv[j], yv[j], ss);
    ss = block_allsum(ss, s_red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    float s2 = 0.0f;
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
        xv[j] += yv[j] * r * (1.0f + bv[j]);
        s2 = fmaf(xv[j], xv[j], s2);
    }
    s2 = block_allsum(s2, s_red);
    const float r2 = 1.0f / sqrtf(s2 / (float)W + eps);
#pragma unroll
    for (int j = 0; j < kRowRegs; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < W) {
            const float h = xv[j] * r2 * (1.0f + nv[j]);
            xr[i] = xv[j];
            out[(size_t)m * W + i] = h + (pv[j] - h) * mv[j];
            if (entry >= 0) last_out[(size_t)entry * W + i] = h;
        }
    }
}

__global__ __launch_bounds__(256) void norm_gather_kernel(const float* x, const int* rows, const float* w, float eps, float* out, int W, float one) {
    __shared__ float s_red[8];
    const int j = blockIdx.x;
    const float* xr = x + (size_t)rows[j] * W;
    const float r = row_inv_rms(xr, W, eps, s_red);
    for (int i = threadIdx.x; i < W; i += blockDim.x) out[(size_t)j * W + i] = xr[i] * r * (one + w[i]);
}

// Side-by-side sublayers: the residual sum the layer before left open, then the two norms of the same row from one statistic.
// Rows of up to 256 * kRowRegs floats stay in registers between the statistic and the results.
__device__ __forceinline__ float open_sums_at(const OpenSums& add, size_t m, int i, int W, float v) {
    if (add.a) v += add.a[m * W + i];
    if (add.exp) {  // in choice order: the sum does not depend on the batch
        float e = 0.0f;
        for (int k = 0; k < add.top; ++k) {
            const float y = add.exp[(m * add.top + k) * W + i];
            e = add.exp_w ? fmaf(add.exp_w[m * add.top + k], y, e) : e + y;
        }
        v += add.b ? e + add.b[m * W + i] : e;
    } else if (add.b) {
        v += add.b[m * W + i];
    }
    if (add.bias) v = fmaf(add.w, add.bias[i], v);
    return v;
}

__global__ __launch_bounds__(256) void norm_two_kernel(float* x, const OpenSums add, const float* wa, const float* wb, float eps, float* ha, float* hb,
                                                       int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    float* xr = x + (size_t)m * W;
    const bool adds = add.any();
    auto value = [&](int i) { return adds ? open_sums_at(add, (size_t)m, i, W, xr[i]) : xr[i]; };
    if (W <= 256 * kRowRegs) {
        float v[kRowRegs];
        float ss = 0.0f;
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            v[j] = i < W ? value(i) : 0.0f;
            ss = fmaf(v[j], v[j], ss);
        }
        ss = block_allsum(ss, s_red);
        const float r = 1.0f / sqrtf(ss / (float)W + eps);
#pragma unroll
        for (int j = 0; j < kRowRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
            if (i < W) {
                if (adds) xr[i] = v[j];
                ha[(size_t)m * W + i] = v[j] * r * wa[i];
                if (hb) hb[(size_t)m * W + i] = v[j] * r * wb[i];
            }
        }
        return;
    }
    float ss = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float v = value(i);
        if (adds) xr[i] = v;  // (each thread reads back only what it wrote itself)
        ss = fmaf(v, v, ss);
    }
    ss = block_allsum(ss, s_red);
    const float r = 1.0f / sqrtf(ss / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        const float v = xr[i];
        ha[(size_t)m * W + i] = v * r * wa[i];
        if (hb) hb[(size_t)m * W + i] = v * r * wb[i];
    }
}

__global__ __launch_bounds__(256) void add_two_kernel(float* x, const OpenSums add, size_t n, int W) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    x[i] = open_sums_at(add, i / W, (int)(i % W), W, x[i]);
}

// one wave per (row, head) vector
__global__ __launch_bounds__(256) void norm_plain_kernel(float* v, int ld, int rows_per_m, int width, int n_vec, const float* w, float eps) {
    const int vec = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (vec >= n_vec) return;
    float* p = v + (size_t)(vec / rows_per_m) * ld + (size_t)(vec % rows_per_m) * width;
    float ss = 0.0f;
    for (int i = lane; i < width; i += 64) ss = fmaf(p[i], p[i], ss);
    ss = wave_allsum(ss);
    const float r = 1.0f / sqrtf(ss / (float)width + eps);
    for (int i = lane; i < width; i += 64) p[i] = p[i] * r * w[i];
}

// ------------------------------------------------------------------------------------------------ norms without statistics
// n(v) = tanh(alpha v) * w + b, nw = [w (W) | b (W) | alpha]: elementwise, so a thread takes four neighbours of a row (rows whose
// width is no multiple of four: one) and every sum around the norm rides in the same pass.
__device__ __forceinline__ float tanh_norm_f(const float* nw, int W, int i, float alpha, float v) { return fmaf(tanhf(alpha * v), nw[i], nw[W + i]); }

template <int VW>
__global__ __launch_bounds__(256) void tanh_norm_kernel(float* x, const float* pre, const float* nw, const int* rows, float* out, size_t n, int W) {
    const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VW;
    if (idx >= n) return;
    const size_t j = idx / W;
    const int i = (int)(idx % W);
    const size_t src = (rows ? (size_t)rows[j] : j) * W + i;
    const float ap = pre ? pre[2 * W] : 0.0f, an = nw ? nw[2 * W] : 0.0f;
    float v[VW];
    if (VW == 4) {
        const f32x4 t = *reinterpret_cast<const f32x4*>(x + src);
        v[0] = t.x; v[VW > 1 ? 1 : 0] = t.y; v[VW > 2 ? 2 : 0] = t.z; v[VW > 3 ? 3 : 0] = t.w;
    } else {
        v[0] = x[src];
    }
    if (pre) {
#pragma unroll
        for (int u = 0; u < VW; ++u) v[u] = tanh_norm_f(pre, W, i + u, ap, v[u]);
        if (VW == 4) *reinterpret_cast<f32x4*>(x + src) = f32x4{v[0], v[VW > 1 ? 1 : 0], v[VW > 2 ? 2 : 0], v[VW > 3 ? 3 : 0]};
        else x[src] = v[0];
    }
    if (!nw) return;
#pragma unroll
    for (int u = 0; u < VW; ++u) v[u] = tanh_norm_f(nw, W, i + u, an, v[u]);
    if (VW == 4) *reinterpret_cast<f32x4*>(out + idx) = f32x4{v[0], v[VW > 1 ? 1 : 0], v[VW > 2 ? 2 : 0], v[VW > 3 ? 3 : 0]};
    else out[idx] = v[0];
}

template <int VW>
__global__ __launch_bounds__(256) void tanh_sum_norm_kernel(float* x, const SumParts y, const float* nb, float mult, const float* nn, float* h, size_t n,
                                                            int W) {
    const size_t idx = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * VW;
    if (idx >= n) return;
    const size_t m = idx / W;
    const int i = (int)(idx % W);
    auto load = [&](const float* p, float* v) {
        if (VW == 4) {
            const f32x4 t = *reinterpret_cast<const f32x4*>(p);
            v[0] = t.x; v[VW > 1 ? 1 : 0] = t.y; v[VW > 2 ? 2 : 0] = t.z; v[VW > 3 ? 3 : 0] = t.w;
        } else {
            v[0] = p[0];
        }
    };
    float a[VW], t[VW], xv[VW];
#pragma unroll
    for (int u = 0; u < VW; ++u) a[u] = 0.0f;
    load(x + idx, xv);
    if (y.a) load(y.a + idx, a);
    for (int k = 0; k < y.top; ++k) {  // in choice order: the sum does not depend on the batch
        const size_t as = m * y.top + k;
        const float wk = y.exp_w ? y.exp_w[as] : 1.0f;
        load(y.exp + (size_t)(y.inv ? y.inv[as] : as) * W + i, t);
#pragma unroll
        for (int u = 0; u < VW; ++u) a[u] = fmaf(wk, t[u], a[u]);
    }
    if (y.b) {
        load(y.b + idx, t);
#pragma unroll
        for (int u = 0; u < VW; ++u) a[u] += t[u];
    }
    const float ab = nb[2 * W], an = nn ? nn[2 * W] : 0.0f;
#pragma unroll
    for (int u = 0; u < VW; ++u) xv[u] = fmaf(mult, tanh_norm_f(nb, W, i + u, ab, a[u]), xv[u]);
    if (VW == 4) *reinterpret_cast<f32x4*>(x + idx) = f32x4{xv[0], xv[VW > 1 ? 1 : 0], xv[VW > 2 ? 2 : 0], xv[VW > 3 ? 3 : 0]};
    else x[idx] = xv[0];
    if (!nn) return;
#pragma unroll
    for (int u = 0; u < VW; ++u) t[u] = tanh_norm_f(nn, W, i + u, an, xv[u]);
    if (VW == 4) *reinterpret_cast<f32x4*>(h + idx) = f32x4{t[0], t[VW > 1 ? 1 : 0], t[VW > 2 ? 2 : 0], t[VW > 3 ? 3 : 0]};
    else h[idx] = t[0];
}

// ------------------------------------------------------------------------------------------------ HGRN2
// A column j of a head's state S[D][V] is held by G consecutive lanes, 16 rows each (D <= 16 G).  The token loop is serial; the
// gates and values of the next SB tokens are staged in the LDS (rows beyond D padded with q = 0, f = 1: they stay zero).
//
// Long entries are cut into chunks of kScanChunk tokens that run side by side (the recurrence is linear in S):
//   phase A   every chunk from a zero state: its end state B_c and the product A_c of its gates per row
//   phase B   S_start(c + 1) = A_c * S_start(c) + B_c down the chunks of an entry (elementwise; S_start overwrites B in place)
//   phase C   every chunk again from its true start state, now writing the outputs
// Short steps (decoding, small portions) run the same kernel once per entry, from the slot's state and back into it.
constexpr int kScanRows = 16;
constexpr int kScanChunk = 64;
enum { SCAN_DIRECT = 0, SCAN_A = 1, SCAN_C = 2 };

// which (entry, chunk) a workgroup of the chunked phases works on; false: none
__device__ __forceinline__ bool scan_find_chunk(int id, const int* ent_len, int n_entries, int& e, int& c) {
    for (e = 0; e < n_entries; ++e) {
        const int nc = (ent_len[e] + kScanChunk - 1) / kScanChunk;
        if (id < nc) {
            c = id;
            return true;
        }
        id -= nc;
    }
    return false;
}

// KIND SCAN_LIN: linear attention with a fixed decay per head on the same layout — the staged "gate" array holds silu(k), the weight of
// the token's value in the state's row, and every row decays by decay[h]:  S <- decay S + k v^T  (q, k, v through silu).
// KIND SCAN_GLA: gated linear attention — q (times a factor), k and v unchanged, and one decay per key channel,
// f = sigmoid(z + bias)^(1 / tau) = exp(log sigmoid(z + bias) / tau) in fp32, staged beside k:  S <- diag(f) S + k v^T.
enum { SCAN_HGRN2 = 0, SCAN_LIN = 1, SCAN_GLA = 2 };
__device__ __forceinline__ float log_sigmoid_f(float z) { return fminf(z, 0.0f) - log1pf(expf(-fabsf(z))); }

template <int G, int KIND>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(const float* proj, int ld, float* out, int ldo, float* state, size_t slot_stride,
                                                         const int* ent_start, const int* ent_len, const int* ent_slot, int n_entries, int H, int D,
                                                         int V, int mode, int SB, float* wsB, float* wsA, const float* bias, const float* low,
                                                         const float* decay, const GlaGate gla) {
    constexpr bool LIN = KIND == SCAN_LIN, GLA = KIND == SCAN_GLA;
    extern __shared__ __attribute__((aligned(16))) float s_scan[];
    constexpr int Dp = G * kScanRows;
    const int cols = blockDim.x / G;
    float* sq = s_scan;             // [SB][Dp]
    float* sf = sq + SB * Dp;       // [SB][Dp]
    float* sv = sf + SB * Dp;       // [SB][cols]
    float* sk = sv + SB * cols;     // [SB][Dp] (SCAN_GLA: the keys; the gate array holds the decays)
    const int h = blockIdx.y;
    const int jl = threadIdx.x / G, g = threadIdx.x % G, j0 = blockIdx.z * cols, j = j0 + jl;
    const bool col_ok = j < V;
    const int HD = H * D;
    int e, c = 0, t_lo, t_hi;
    if (mode == SCAN_DIRECT) {
        e = blockIdx.x;
        t_lo = 0;
        t_hi = ent_len[e];
    } else {
        if (!scan_find_chunk(blockIdx.x, ent_len, n_entries, e, c)) return;
        t_lo = c * kScanChunk;
        t_hi = min(ent_len[e], t_lo + kScanChunk);
    }
    const int m0 = ent_start[e];
    const size_t head_floats = (size_t)D * V;
    const float dec = LIN ? decay[h] : 0.0f;
    float* S_slot = state + (size_t)ent_slot[e] * slot_stride + (size_t)h * head_floats;
    float* S_ws = wsB ? wsB + ((size_t)blockIdx.x * H + h) * head_floats : nullptr;
    const float* S_in = mode == SCAN_DIRECT ? S_slot : mode == SCAN_C ? S_ws : nullptr;
    float S[kScanRows], A[kScanRows];
#pragma unroll
    for (int r = 0; r < kScanRows; ++r) {
        const int i = g * kScanRows + r;
        S[r] = (S_in && col_ok && i < D) ? S_in[(size_t)i * V + j] : 0.0f;
        A[r] = 1.0f;
    }
    for (int tb = t_lo; tb < t_hi; tb += SB) {
        const int nb = min(SB, t_hi - tb);
        __syncthreads();  // the previous block has been consumed
        for (int idx = threadIdx.x; idx < nb * Dp; idx += blockDim.x) {
            const int tt = idx / Dp, i = idx % Dp;
            const float* row = proj + (size_t)(m0 + tb + tt) * ld;
            // the gates are activated on their way into the LDS: q = silu(.), f = low + (1 - low) sigmoid(. + bias)
            float qv = 0.0f, fv = LIN ? 0.0f : 1.0f, kv = 0.0f;
            if (i < D) {
                if (GLA) {
                    qv = row[h * D + i] * gla.q_scale;
                    kv = row[HD + h * D + i];
                    fv = expf(log_sigmoid_f(gla.z[(size_t)(m0 + tb + tt) * gla.ldz + h * D + i] + gla.z_bias[h * D + i]) * gla.inv_tau);
                } else {
                    qv = silu_f(row[h * D + i]);
                    if (LIN) {
                        fv = silu_f(row[HD + h * D + i]);
                    } else {
                        const float l = low[h * D + i];
                        fv = l + (1.0f - l) * sigmoid_f(row[HD + h * D + i] + bias[h * D + i]);
                    }
                }
            }
            sq[idx] = qv;
            sf[idx] = fv;
            if (GLA) sk[idx] = kv;
        }
        for (int idx = threadIdx.x; idx < nb * cols; idx += blockDim.x) {
            const int tt = idx / cols, jj = idx % cols;
            const float vin = j0 + jj < V ? proj[(size_t)(m0 + tb + tt) * ld + 2 * HD + h * V + j0 + jj] : 0.0f;
            sv[idx] = LIN ? silu_f(vin) : vin;
        }
        __syncthreads();
        for (int tt = 0; tt < nb; ++tt) {
            const f32x4* q4 = reinterpret_cast<const f32x4*>(sq + tt * Dp + g * kScanRows);
            const f32x4* f4 = reinterpret_cast<const f32x4*>(sf + tt * Dp + g * kScanRows);
            const f32x4* k4 = reinterpret_cast<const f32x4*>(sk + tt * Dp + g * kScanRows);
            const float v = sv[tt * cols + jl];
            float o = 0.0f;
#pragma unroll
            for (int r4 = 0; r4 < kScanRows / 4; ++r4) {
                const f32x4 qq = q4[r4], ff = f4[r4];
                const f32x4 kk = GLA ? k4[r4] : ff;
                const float qv[4] = {qq.x, qq.y, qq.z, qq.w}, fv[4] = {ff.x, ff.y, ff.z, ff.w}, kv[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int r = r4 * 4 + u;
                    S[r] = GLA ? fmaf(fv[u], S[r], kv[u] * v) : LIN ? fmaf(dec, S[r], fv[u] * v) : fmaf(fv[u], S[r], (1.0f - fv[u]) * v);
                    o = fmaf(S[r], qv[u], o);
                    if (mode == SCAN_A) A[r] *= LIN ? dec : fv[u];
                }
            }
            if (mode != SCAN_A) {
#pragma unroll
                for (int off = 1; off < G; off <<= 1) o += __shfl_xor(o, off, 64);
                if (g == 0 && col_ok) out[(size_t)(m0 + tb + tt) * ldo + h * V + j] = o;
            }
        }
    }
    float* S_out = mode == SCAN_DIRECT ? S_slot : mode == SCAN_A ? S_ws : nullptr;
    if (S_out) {
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) {
            const int i = g * kScanRows + r;
            if (col_ok && i < D) S_out[(size_t)i * V + j] = S[r];
        }
    }
    if (mode == SCAN_A && blockIdx.z == 0 && jl == 0) {
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) {
            const int i = g * kScanRows + r;
            if (i < D) wsA[((size_t)blockIdx.x * H + h) * D + i] = A[r];
        }
    }
}

// phase B: one thread per state element walks the chunks of its entry
__global__ __launch_bounds__(256) void hgrn2_carry_kernel(float* state, size_t slot_stride, const int* ent_len, const int* ent_slot, int n_entries, int H,
                                                          int D, int V, float* wsB, const float* wsA, int chunk) {
    const int e = blockIdx.y;
    const size_t n = (size_t)H * D * V, idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    int first = 0;
    for (int k = 0; k < e; ++k) first += (ent_len[k] + chunk - 1) / chunk;
    const int nc = (ent_len[e] + chunk - 1) / chunk;
    const size_t hi = idx / V;  // (head, row)
    float* slot = state + (size_t)ent_slot[e] * slot_stride;
    float S = slot[idx];
    for (int c0 = 0; c0 < nc; c0 += 8) {  // eight chunks' operands requested together: the chain itself is eight multiply-adds
        float Bv[8], Av[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = min(c0 + u, nc - 1);
            Bv[u] = wsB[(size_t)(first + c) * n + idx];
            Av[u] = wsA[(size_t)(first + c) * H * D + hi];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c0 + u < nc) {
                wsB[(size_t)(first + c0 + u) * n + idx] = S;  // the chunk's start state for phase C
                S = fmaf(Av[u], S, Bv[u]);
            }
    }
    if (nc > 0) slot[idx] = S;
}

// ------------------------------------------------------------------------------------------------ linear attention, chunks on the matrix cores
// With ONE decay per head the recurrence S <- lambda S + k v^T, o = S^T q of a chunk of n <= 32 tokens is three matrix products
// (true fp32, v_mfma_f32_32x32x2_f32; q, k, v through silu on load):
//   state   B = sum_j lambda^(n-1-j) k_j v_j^T                       the chunk's end state from zero          (phase A, per chunk)
//   carry   S_start(c + 1) = lambda^n S_start(c) + B_c               down the chunks of an entry              (hgrn2_carry_kernel)
//   output  o_i = sum_(j<=i) lambda^(i-j) (q_i . k_j) v_j + lambda^(i+1) S_start^T q_i                        (phase C, per chunk)
// A workgroup takes a (chunk, head); lane (r, half) of a wave holds channels half * Dh .. of row r (the order inside a dot product
// is free), tokens half * 16 .. where the tokens are the product's inner dimension.
constexpr int kLinChunk = 32;
typedef __attribute__((ext_vector_type(16))) float f32x16_lin;

__device__ __forceinline__ float decay_pow(float lam, float l2, int n) { return n <= 0 ? 1.0f : (lam <= 0.0f ? 0.0f : exp2f((float)n * l2)); }

__device__ __forceinline__ bool lin_find_chunk(int id, const int* ent_len, int n_entries, int& e, int& c) {
    for (e = 0; e < n_entries; ++e) {
        const int nc = (ent_len[e] + kLinChunk - 1) / kLinChunk;
        if (id < nc) {
            c = id;
            return true;
        }
        id -= nc;
    }
    return false;
}

__global__ __launch_bounds__(256) void linear_chunk_state_kernel(const float* __restrict__ proj, int ld, const int* ent_start, const int* ent_len,
                                                                 int n_entries, int H, int D, int V, const float* decay, float* __restrict__ wsB,
                                                                 float* __restrict__ wsA) {
    int e, c;
    if (!lin_find_chunk(blockIdx.x, ent_len, n_entries, e, c)) return;
    const int h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, kh = lane >> 5;
    const int n = min(kLinChunk, ent_len[e] - c * kLinChunk), m0 = ent_start[e] + c * kLinChunk, HD = H * D;
    const float lam = decay[h], l2 = lam > 0.0f ? log2f(lam) : 0.0f;
    const float* kbase = proj + (size_t)m0 * ld + HD + (size_t)h * D;
    const float* vbase = proj + (size_t)m0 * ld + 2 * HD + (size_t)h * V;
    float* B = wsB + ((size_t)blockIdx.x * H + h) * D * V;
    const int tilesD = (D + 31) / 32, tilesV = (V + 31) / 32;
    for (int tile = blockIdx.z * 4 + wave; tile < tilesD * tilesV; tile += 4 * gridDim.z) {
        const int d0 = (tile / tilesV) * 32, v0 = (tile % tilesV) * 32;
        float a[16], b[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {  // token j is the inner dimension: weight lambda^(n - 1 - j) on the key
            const int j = kh * 16 + t;
            a[t] = (j < n && d0 + r < D) ? kbase[(size_t)j * ld + d0 + r] : 0.0f;
            b[t] = (j < n && v0 + r < V) ? vbase[(size_t)j * ld + v0 + r] : 0.0f;
        }
        f32x16_lin acc;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; ++t)
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(silu_f(a[t]) * decay_pow(lam, l2, n - 1 - (kh * 16 + t)), silu_f(b[t]), acc, 0, 0, 0);
        // accumulator element i: row 8 (i / 4) + 4 half + i % 4, column r
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int d = d0 + 8 * (i >> 2) + 4 * kh + (i & 3);
            if (d < D && v0 + r < V) B[(size_t)d * V + v0 + r] = acc[i];
        }
    }
    if (blockIdx.z == 0)
        for (int i = threadIdx.x; i < D; i += blockDim.x) wsA[((size_t)blockIdx.x * H + h) * D + i] = decay_pow(lam, l2, n);
}

template <int DH>
__global__ __launch_bounds__(256) void linear_chunk_out_kernel(const float* __restrict__ proj, int ld, float* __restrict__ out, int ldo,
                                                               const int* ent_start, const int* ent_len, int n_entries, int H, int D, int V,
                                                               const float* decay, const float* __restrict__ wsB) {
    __shared__ float s_p[4][32][33];
    int e, c;
    if (!lin_find_chunk(blockIdx.x, ent_len, n_entries, e, c)) return;
    const int h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, kh = lane >> 5;
    const int n = min(kLinChunk, ent_len[e] - c * kLinChunk), m0 = ent_start[e] + c * kLinChunk, HD = H * D, Dh = (D + 1) / 2;
    const float lam = decay[h], l2 = lam > 0.0f ? log2f(lam) : 0.0f;
    const float* S = wsB + ((size_t)blockIdx.x * H + h) * D * V;  // the chunk's start state (the carry left it here)
    const float* qrow = proj + (size_t)(m0 + min(r, n - 1)) * ld + (size_t)h * D + kh * Dh;
    const float* krow = qrow + HD;
    const float* vbase = proj + (size_t)m0 * ld + 2 * HD + (size_t)h * V;
    float qreg[DH], kreg[DH];
    // 16-byte loads where a lane's run of channels starts on a 16-byte boundary and is a multiple of four long
    const bool vec = D % 8 == 0 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(proj) & 15) == 0;
    if (vec) {
#pragma unroll
        for (int t = 0; t < DH; t += 4) {
            const bool ok = r < n && t < Dh;
            const f32x4 a = ok ? *reinterpret_cast<const f32x4*>(qrow + t) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const f32x4 b = ok ? *reinterpret_cast<const f32x4*>(krow + t) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            qreg[t] = a.x; qreg[t + 1] = a.y; qreg[t + 2] = a.z; qreg[t + 3] = a.w;
            kreg[t] = b.x; kreg[t + 1] = b.y; kreg[t + 2] = b.z; kreg[t + 3] = b.w;
        }
    } else {
#pragma unroll
        for (int t = 0; t < DH; ++t) {
            const bool ok = r < n && t < Dh && kh * Dh + t < D;
            qreg[t] = ok ? qrow[t] : 0.0f;
            kreg[t] = ok ? krow[t] : 0.0f;
        }
    }
#pragma unroll
    for (int t = 0; t < DH; ++t) {
        qreg[t] = silu_f(qreg[t]);
        kreg[t] = silu_f(kreg[t]);
    }
    f32x16_lin acc;
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
    for (int t = 0; t < DH; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[t], kreg[t], acc, 0, 0, 0);
    // element i: query 8 (i / 4) + 4 half + i % 4, key r: the decay of their distance, nothing for keys behind the query
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const int qi = 8 * (i >> 2) + 4 * kh + (i & 3);
        s_p[wave][qi][r] = (r <= qi && qi < n) ? acc[i] * decay_pow(lam, l2, qi - r) : 0.0f;
    }
    __syncthreads();
    const float carry = decay_pow(lam, l2, r + 1);  // what the start state has decayed to when token r reads it
#pragma unroll
    for (int t = 0; t < DH; ++t) qreg[t] *= carry;
    const int tilesV = (V + 31) / 32;
    for (int vt = wave; vt < tilesV; vt += 4) {
        const int v0 = vt * 32;
        const bool col_ok = v0 + r < V;
        float vv[16];
#pragma unroll
        for (int t = 0; t < 16; ++t) {
            const int j = kh * 16 + t;
            vv[t] = (j < n && col_ok) ? vbase[(size_t)j * ld + v0 + r] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
        for (int t = 0; t < 16; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(s_p[wave][r][kh * 16 + t], silu_f(vv[t]), acc, 0, 0, 0);
#pragma unroll
        for (int t0 = 0; t0 < DH; t0 += 16) {  // the start state's share, 16 state rows requested at a time
            float sv[16];
#pragma unroll
            for (int u = 0; u < 16; ++u) {
                const int t = t0 + u, ch = kh * Dh + t;
                sv[u] = (t < DH && t < Dh && ch < D && col_ok) ? S[(size_t)ch * V + v0 + r] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 16; ++u)
                if (t0 + u < DH) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[min(t0 + u, DH - 1)], sv[u], acc, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int qi = 8 * (i >> 2) + 4 * kh + (i & 3);
            if (qi < n && col_ok) out[(size_t)(m0 + qi) * ldo + (size_t)h * V + v0 + r] = acc[i];
        }
    }
}

// ------------------------------------------------------------------------------------------------ latent attention
__device__ __forceinline__ size_t cache_row(const int* page_table, int max_pages, int page_tokens, int slot, int pos) {
    return (size_t)page_table[(size_t)slot * max_pages + pos / page_tokens] * page_tokens + pos % page_tokens;
}

// the interleaved pair (2i, 2i + 1) of `src` at position pos, rotated by pos * freq[i]; angle and product in fp32
__device__ __forceinline__ void rotate_pair(const float* src, float* dst, int i, int pos, const Rotary& rot) {
    const float a = (float)pos * rot.freq[i];
    const float c = cosf(a) * rot.amp, s = sinf(a) * rot.amp;
    const float u = src[2 * i], v = src[2 * i + 1];
    dst[2 * i] = u * c - v * s;
    dst[2 * i + 1] = v * c + u * s;
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const float* proj, int ld, int q_rank, int KR, int R, const float* wq, const float* wkv,
                                                          float eps, Rotary rot, const int* row_pos, const int* row_slot, const int* page_table,
                                                          int max_pages, int page_tokens, float* cq, float* cache) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float* row = proj + (size_t)m * ld;
    const float rq = row_inv_rms(row, q_rank, eps, s_red);
    const float rc = row_inv_rms(row + q_rank, KR, eps, s_red);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cq[(size_t)m * q_rank + i] = row[i] * rq * wq[i];
    const int pos = row_pos[m];
    float* crow = cache + cache_row(page_table, max_pages, page_tokens, row_slot[m], pos) * (size_t)(KR + R);
    for (int i = threadIdx.x; i < KR; i += blockDim.x) crow[i] = row[q_rank + i] * rc * wkv[i];
    const float* kr = row + q_rank + KR;
    for (int i = threadIdx.x; i < rot.dims / 2; i += blockDim.x) rotate_pair(kr, crow + KR, i, pos, rot);
    for (int i = rot.dims + threadIdx.x; i < R; i += blockDim.x) crow[KR + i] = kr[i];
}

__global__ __launch_bounds__(256) void q_rotary_kernel(const float* q, int ldq, float* qa, int ldqa, int H, int D, int R, int KR, Rotary rot,
                                                       const int* row_pos) {
    const int m = blockIdx.x, pos = row_pos[m], half = rot.dims / 2;
    for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
        const int h = idx / half, i = idx % half;
        rotate_pair(q + (size_t)m * ldq + (size_t)h * (D + R) + D, qa + (size_t)m * ldqa + (size_t)h * (KR + R) + KR, i, pos, rot);
    }
    const int rest = R - rot.dims;
    for (int idx = threadIdx.x; idx < H * rest; idx += blockDim.x) {
        const int h = idx / rest, i = rot.dims + idx % rest;
        qa[(size_t)m * ldqa + (size_t)h * (KR + R) + KR + i] = q[(size_t)m * ldq + (size_t)h * (D + R) + D + i];
    }
}

// One workgroup per (row, head).  The lanes of a wave split the KR + R dimensions of a cache row (ND per lane); a wave walks
// its share of the keys four at a time with a running (maximum, sum, weighted latent) and the four waves are merged at the end.
// With n_split > 1 (decode steps: few rows, long key ranges) grid.z workgroups share a row's keys in ranges of at least 64
// and leave (maximum, sum, weighted latent) partials in ws for latent_merge_kernel.
template <int ND>
__global__ __launch_bounds__(256) void latent_attention_kernel(const float* qa, float* ctx, int H, int KR, int R, float scale, const int* row_pos,
                                                               const int* row_slot, const int* page_table, int max_pages, int page_tokens,
                                                               const float* cache, float* ws, int n_split) {
    __shared__ float s_m[4], s_l[4];
    __shared__ float s_acc[4][ND * 64];
    const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int DT = KR + R, n_keys = row_pos[m] + 1, slot = row_slot[m];
    int k_lo = 0, k_hi = n_keys;
    if (n_split > 1) {
        int chunk = (n_keys + n_split - 1) / n_split;
        chunk = max(64, (chunk + 15) & ~15);
        k_lo = min(n_keys, (int)blockIdx.z * chunk);
        k_hi = min(n_keys, k_lo + chunk);
    }
    const float* qrow = qa + ((size_t)m * H + h) * DT;
    float q[ND], acc[ND];
#pragma unroll
    for (int i = 0; i < ND; ++i) {
        const int d = lane + 64 * i;
        q[i] = d < DT ? qrow[d] : 0.0f;
        acc[i] = 0.0f;
    }
    float mx = -INFINITY, l = 0.0f;
    const int* pt = page_table + (size_t)slot * max_pages;
    for (int kb = k_lo + wave * 4; kb < k_hi; kb += 16) {
        float r[4][ND], s[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int key = kb + u < k_hi ? kb + u : kb;
            const float* row = cache + ((size_t)pt[key / page_tokens] * page_tokens + key % page_tokens) * DT;
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < ND; ++i) {
                const int d = lane + 64 * i;
                r[u][i] = d < DT ? row[d] : 0.0f;
                part = fmaf(q[i], r[u][i], part);
            }
            s[u] = part;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            s[u] = wave_allsum(s[u]) * scale;
            if (kb + u >= k_hi) s[u] = -INFINITY;
        }
        const float mn = fmaxf(fmaxf(mx, s[0]), fmaxf(fmaxf(s[1], s[2]), s[3]));
        const float alpha = expf(mx - mn);  // 0 for the first group (mx = -inf, mn finite: key kb is always valid)
        float pw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) pw[u] = expf(s[u] - mn);
        l = l * alpha + ((pw[0] + pw[1]) + (pw[2] + pw[3]));
#pragma unroll
        for (int i = 0; i < ND; ++i) {
            float a = acc[i] * alpha;
#pragma unroll
            for (int u = 0; u < 4; ++u) a = fmaf(pw[u], r[u][i], a);
            acc[i] = a;
        }
        mx = mn;
    }
    if (lane == 0) {
        s_m[wave] = mx;
        s_l[wave] = l;
    }
#pragma unroll
    for (int i = 0; i < ND; ++i) s_acc[wave][lane + 64 * i] = acc[i];
    __syncthreads();
    const float M4 = fmaxf(fmaxf(s_m[0], s_m[1]), fmaxf(s_m[2], s_m[3]));
    float wgt[4], L = 0.0f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        wgt[w] = M4 == -INFINITY ? 0.0f : expf(s_m[w] - M4);  // a wave without keys: exp(-inf) = 0; a range without keys: all zero
        L += wgt[w] * s_l[w];
    }
    if (n_split > 1) {
        float* part = ws + (((size_t)m * H + h) * n_split + blockIdx.z) * (KR + 2);
        if (threadIdx.x == 0) {
            part[0] = M4;
            part[1] = L;
        }
        for (int d = threadIdx.x; d < KR; d += blockDim.x) {
            float a = 0.0f;
#pragma unroll
            for (int w = 0; w < 4; ++w) a = fmaf(wgt[w], s_acc[w][d], a);
            part[2 + d] = a;
        }
        return;
    }
    float* out = ctx + ((size_t)m * H + h) * KR;
    for (int d = threadIdx.x; d < KR; d += blockDim.x) {
        float a = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) a = fmaf(wgt[w], s_acc[w][d], a);
        out[d] = a / L;
    }
}

// Prompt portions in bf16 mode: the same attention on the matrix cores.  A workgroup takes 32 consecutive queries of one entry
// and four heads (one per wave) — the heads share the cached rows, so a tile of 32 keys is staged in the LDS once for all four:
// as bf16 rows [key][dim] for the scores and, its latent part, transposed [dim][key] for the weighted sum.  Both products are
// computed transposed (S^T = K Q^T, O^T = C^T P^T): a lane's column is a query, so the running maximum and sum are per-lane
// values and the probabilities a lane computed are exactly the eight per k-step it has to feed back (in a key order that the
// transposed latent tile is read in as well: keys {0-3, 8-11} from the lower half-wave, {4-7, 12-15} from the upper one).
// Scores, softmax and both accumulations are fp32; q, cache rows and probabilities enter the products as bf16.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <int NKS, int NT>  // 16 NKS >= KR + R (score dimensions), 32 NT >= KR (latent dimensions)
__global__ __launch_bounds__(256) void latent_attention_mfma_kernel(const float* qa, float* ctx, int H, int KR, int R, float scale,
                                                                    const int* ent_start, const int* ent_len, const int* ent_slot, int n_entries,
                                                                    const int* row_pos, const int* page_table, int max_pages, int page_tokens,
                                                                    const float* cache) {
    constexpr int DTp = NKS * 16, KS_LD = DTp + 8, VT_LD = 40;
    __shared__ __attribute__((aligned(16))) bf16_t Ks[32 * KS_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Vt[NT * 32 * VT_LD];
    int id = blockIdx.x, e = 0, qb = 0;
    for (; e < n_entries; ++e) {
        const int nb = (ent_len[e] + 31) / 32;
        if (id < nb) {
            qb = id;
            break;
        }
        id -= nb;
    }
    if (e >= n_entries) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, hf = lane >> 5;
    const int h = blockIdx.y * 4 + wave;
    const bool head_ok = h < H;
    const int m_first = ent_start[e] + qb * 32, nq = min(32, ent_len[e] - qb * 32);
    const int pos_first = row_pos[m_first], qpos = pos_first + r, DT = KR + R;
    const bool q_ok = r < nq;
    const int n_keys = pos_first + nq;
    const int* pt = page_table + (size_t)ent_slot[e] * max_pages;

    bf16x8 qf[NKS];
    {
        const float* qrow = qa + ((size_t)(m_first + (q_ok ? r : 0)) * H + (head_ok ? h : 0)) * DT;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int d = ks * 16 + 8 * hf + u;
                v[u] = (head_ok && q_ok && d < DT) ? qrow[d] : 0.0f;
            }
            u32x4 pk;
            pk.x = cvt_pk_bf16(v[0], v[1]);
            pk.y = cvt_pk_bf16(v[2], v[3]);
            pk.z = cvt_pk_bf16(v[4], v[5]);
            pk.w = cvt_pk_bf16(v[6], v[7]);
            qf[ks] = __builtin_bit_cast(bf16x8, pk);
        }
    }
    f32x16 o[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[t][i] = 0.0f;
    float mx = -INFINITY, lsum = 0.0f;
    const bool vec = (DT % 4 == 0) && ((reinterpret_cast<uintptr_t>(cache) & 15) == 0);

    // a tile's rows travel global -> registers -> LDS; the registers of tile kt + 1 are filled while tile kt is multiplied
    constexpr int ITEMS = 32 * (DTp / 4) / 256;  // float4 pieces per thread and tile (NKS is even)
    f32x4 stage[ITEMS];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            const int idx = tid + 256 * it;
            const int key = idx / (DTp / 4), d4 = (idx % (DTp / 4)) * 4, kpos = kt * 32 + key;
            f32x4 x = {0.0f, 0.0f, 0.0f, 0.0f};
            if (kpos < n_keys) {
                const float* row = cache + ((size_t)pt[kpos / page_tokens] * page_tokens + kpos % page_tokens) * DT;
                if (vec && d4 + 4 <= DT) {
                    x = *reinterpret_cast<const f32x4*>(row + d4);
                } else {
                    x.x = d4 + 0 < DT ? row[d4 + 0] : 0.0f;
                    x.y = d4 + 1 < DT ? row[d4 + 1] : 0.0f;
                    x.z = d4 + 2 < DT ? row[d4 + 2] : 0.0f;
                    x.w = d4 + 3 < DT ? row[d4 + 3] : 0.0f;
                }
            }
            stage[it] = x;
        }
    };
    fetch(0);
    for (int kt = 0; kt * 32 < n_keys; ++kt) {
        __syncthreads();  // the previous tile has been consumed
#pragma unroll
        for (int it = 0; it < ITEMS; ++it) {
            const int idx = tid + 256 * it;
            const int key = idx / (DTp / 4), d4 = (idx % (DTp / 4)) * 4;
            u32x2 pk;
            pk.x = cvt_pk_bf16(stage[it].x, stage[it].y);
            pk.y = cvt_pk_bf16(stage[it].z, stage[it].w);
            *reinterpret_cast<u32x2*>(&Ks[key * KS_LD + d4]) = pk;
        }
        __syncthreads();
        if ((kt + 1) * 32 < n_keys) fetch(kt + 1);
        // the latent part once more, transposed: consecutive lanes take consecutive keys, so the 2-byte stores of a wave fall into
        // consecutive words (written from the rows above rather than beside them: a lane of the loop above holds four dimensions
        // of ONE key, and its four stores would all hit the same two banks)
        for (int idx = tid; idx < 32 * (NT * 8); idx += 256) {
            const int key = idx & 31, d4 = (idx >> 5) * 4;
            const u32x2 pk = *reinterpret_cast<const u32x2*>(&Ks[key * KS_LD + d4]);
            Vt[(d4 + 0) * VT_LD + key] = (bf16_t)(pk.x & 0xFFFFu);
            Vt[(d4 + 1) * VT_LD + key] = (bf16_t)(pk.x >> 16);
            Vt[(d4 + 2) * VT_LD + key] = (bf16_t)(pk.y & 0xFFFFu);
            Vt[(d4 + 3) * VT_LD + key] = (bf16_t)(pk.y >> 16);
        }
        __syncthreads();
        if (!head_ok) continue;
        f32x16 sacc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const bf16x8 a = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Ks[r * KS_LD + ks * 16 + 8 * hf]));
            sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], sacc, 0, 0, 0);
        }
        float sv[16], tmax = -INFINITY;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int key = kt * 32 + 8 * (i >> 2) + 4 * hf + (i & 3);
            sv[i] = (q_ok && key <= qpos) ? sacc[i] * scale : -INFINITY;
            tmax = fmaxf(tmax, sv[i]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        // The reference point of the exponentials moves only when some query's maximum grew by more than 8 (the weights then
        // reach e^8 at most, far inside fp32 and bf16 range): the accumulators are rescaled on few tiles instead of on every one.
        const bool grow = tmax > mx + 8.0f;  // also the first tile of a query (mx = -inf)
        float psum = 0.0f, pv[16];
        if (__any(grow)) {
            const float mn = grow ? tmax : mx;
            const float alpha = (mn == -INFINITY || mx == mn) ? 1.0f : __expf(mx - mn);  // mx = -inf, mn finite: 0
            lsum *= alpha;
#pragma unroll
            for (int t = 0; t < NT; ++t)
#pragma unroll
                for (int i = 0; i < 16; ++i) o[t][i] *= alpha;
            mx = mn;
        }
        const bool none = mx == -INFINITY;  // a query row beyond the entry: nothing to weigh
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            pv[i] = none ? 0.0f : __expf(sv[i] - mx);
            psum += pv[i];
        }
        lsum += psum;
        u32x4 p0, p1;
        p0.x = cvt_pk_bf16(pv[0], pv[1]); p0.y = cvt_pk_bf16(pv[2], pv[3]); p0.z = cvt_pk_bf16(pv[4], pv[5]); p0.w = cvt_pk_bf16(pv[6], pv[7]);
        p1.x = cvt_pk_bf16(pv[8], pv[9]); p1.y = cvt_pk_bf16(pv[10], pv[11]); p1.z = cvt_pk_bf16(pv[12], pv[13]); p1.w = cvt_pk_bf16(pv[14], pv[15]);
        const bf16x8 pf0 = __builtin_bit_cast(bf16x8, p0), pf1 = __builtin_bit_cast(bf16x8, p1);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            const bf16_t* vrow = &Vt[(t * 32 + r) * VT_LD + 4 * hf];
            const u32x2 a0 = *reinterpret_cast<const u32x2*>(vrow), a1 = *reinterpret_cast<const u32x2*>(vrow + 8);
            const u32x2 b0 = *reinterpret_cast<const u32x2*>(vrow + 16), b1 = *reinterpret_cast<const u32x2*>(vrow + 24);
            o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, (u32x4){a0.x, a0.y, a1.x, a1.y}), pf0, o[t], 0, 0, 0);
            o[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, (u32x4){b0.x, b0.y, b1.x, b1.y}), pf1, o[t], 0, 0, 0);
        }
    }
    if (!head_ok) return;
    const float L = lsum + __shfl_xor(lsum, 32, 64);
    if (!q_ok) return;
    float* out = ctx + ((size_t)(m_first + r) * H + h) * KR;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int d = t * 32 + 8 * (i >> 2) + 4 * hf + (i & 3);
            if (d < KR) out[d] = o[t][i] / L;
        }
}

// ctx[m][h] from the partials of latent_attention_kernel, in a fixed order (the result does not depend on timing); only the
// ranges that held keys are read
__global__ __launch_bounds__(256) void latent_merge_kernel(const float* ws, float* ctx, int H, int KR, int n_split, const int* row_pos) {
    __shared__ float s_w[64];
    __shared__ float s_L;
    const int m = blockIdx.x, h = blockIdx.y, n_keys = row_pos[m] + 1;
    int chunk = (n_keys + n_split - 1) / n_split;
    chunk = max(64, (chunk + 15) & ~15);
    const int used = min(n_split, (n_keys + chunk - 1) / chunk);
    const float* part = ws + ((size_t)m * H + h) * n_split * (KR + 2);
    if (threadIdx.x < 64) {
        const int sidx = threadIdx.x;
        const float pm = sidx < used ? part[(size_t)sidx * (KR + 2)] : -INFINITY;
        const float M = wave_allmax(pm);
        const float w = pm == -INFINITY ? 0.0f : expf(pm - M);
        s_w[sidx] = w;
        const float L = wave_allsum(sidx < used ? w * part[(size_t)sidx * (KR + 2) + 1] : 0.0f);
        if (sidx == 0) s_L = L;
    }
    __syncthreads();
    float* out = ctx + ((size_t)m * H + h) * KR;
    const float L = s_L;
    for (int d = threadIdx.x; d < KR; d += blockDim.x) {
        float a = 0.0f;
        for (int sidx = 0; sidx < used; ++sidx) a = fmaf(s_w[sidx], part[(size_t)sidx * (KR + 2) + 2 + d], a);
        out[d] = a / L;
    }
}

// Stage 1: block (row, part) finds the maximum and its first index in its slice of the row; stage 2 (parts == 1 in the grid,
// n_parts > 0 as argument): one block per row combines the parts.  The first maximum wins; a row of NaNs gives index 0.
__global__ __launch_bounds__(256) void row_argmax_kernel(const float* logits, int n, float* max_out, int* idx_out, float* part_val, int* part_idx,
                                                         int n_parts, int combine) {
    __shared__ float s_v[4];
    __shared__ int s_i[4];
    const int row = blockIdx.x;
    float best = -INFINITY;
    int bi = 0x7fffffff;
    if (!combine) {
        const int per = (n + n_parts - 1) / n_parts, lo = blockIdx.y * per, hi = min(n, lo + per);
        const float* r = logits + (size_t)row * n;
        for (int i = lo + threadIdx.x; i < hi; i += blockDim.x) {
            const float v = r[i];
            if (v > best) {  // ascending i per thread: the first maximum stays
                best = v;
                bi = i;
            }
        }
    } else {
        for (int i = threadIdx.x; i < n_parts; i += blockDim.x) {
            const float v = part_val[(size_t)row * n_parts + i];
            const int ix = part_idx[(size_t)row * n_parts + i];
            if (v > best || (v == best && ix < bi)) {
                best = v;
                bi = ix;
            }
        }
    }
    const float wbest = wave_allmax(best);
    int cand = (best == wbest) ? bi : 0x7fffffff;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) cand = min(cand, __shfl_xor(cand, off, 64));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        s_v[wave] = wbest;
        s_i[wave] = cand;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float v = s_v[0];
        int ix = s_i[0];
        for (int w = 1; w < 4; ++w)
            if (s_v[w] > v || (s_v[w] == v && s_i[w] < ix)) {
                v = s_v[w];
                ix = s_i[w];
            }
        if (!combine) {
            part_val[(size_t)row * n_parts + blockIdx.y] = v;
            part_idx[(size_t)row * n_parts + blockIdx.y] = ix;
        } else {
            if (ix == 0x7fffffff) ix = 0;
            if (max_out) max_out[row] = v;
            if (idx_out) idx_out[row] = ix;
        }
    }
}

}  // namespace

int launch_embed(const bf16_t* table, const int* ids, float* x, float* x_copy, float scale, int M, int W, int vocab, int* flag, const int* row_pos,
                 const float* pos_freq, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    embed_kernel<<<M, 256, 0, s>>>(table, ids, x, x_copy, scale, W, vocab, flag, pos_freq ? row_pos : nullptr, pos_freq);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_shift(const float* x, const float* w, const float* mu, float eps, float* out, int M, int W, const int* row_prev,
                      const int* row_slot, const float* shift_state, size_t slot_stride, const int* row_entry_if_last, float* last_out,
                      hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_shift_kernel<<<M, 256, 0, s>>>(x, w, mu, eps, out, W, row_prev, row_slot, shift_state, slot_stride, row_entry_if_last, last_out);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_commit_rows(float* dst, size_t slot_stride, const float* src, size_t src_stride, const int* slots, int n_entries, int width,
                       int n_sets, size_t dst_set_stride, size_t src_set_stride, hipStream_t s) {
    if (n_entries <= 0 || n_sets <= 0) return ZG_OK;
    commit_rows_kernel<<<dim3(n_entries, n_sets), 256, 0, s>>>(dst, slot_stride, src, src_stride, slots, width, dst_set_stride, src_set_stride);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_add(float* x, const float* y, const float* w, float eps, int M, int W, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_add_kernel<<<M, 256, 0, s>>>(x, y, w, eps, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_add_norm(float* x, const float* y, const float* wb, const float* wn, float eps, float* h, int M, int W, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_add_norm_kernel<<<M, 256, 0, s>>>(x, y, wb, wn, eps, h, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_sum_norm_shift(float* x, const float* y, const float* yexp, const float* weight, int top, const float* wb, const float* wn, const float* mu,
                          float eps, float* out, int M, int W, const int* row_slot, const float* shift_state, size_t slot_stride,
                          const int* row_entry_if_last, float* last_out, hipStream_t s, bool* taken) {
    *taken = false;
    if (M <= 0 || W > 256 * kRowRegs) return ZG_OK;  // wider rows: the caller's separate launches
    sum_norm_shift_kernel<<<M, 256, 0, s>>>(x, y, yexp, weight, top, wb, wn, mu, eps, out, W, row_slot, shift_state, slot_stride, row_entry_if_last,
                                            last_out);
    ZG_HIP(hipGetLastError());
    *taken = true;
    return ZG_OK;
}

int launch_norm_gather(const float* x, const int* rows, const float* w, float eps, float* out, int n_rows, int W, bool plain, hipStream_t s) {
    if (n_rows <= 0) return ZG_OK;
    norm_gather_kernel<<<n_rows, 256, 0, s>>>(x, rows, w, eps, out, W, plain ? 0.0f : 1.0f);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_two(float* x, const OpenSums& add, const float* wa, const float* wb, float eps, float* ha, float* hb, int M, int W, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    norm_two_kernel<<<M, 256, 0, s>>>(x, add, wa, wb, eps, ha, wb ? hb : nullptr, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_add_two(float* x, const OpenSums& add, int M, int W, hipStream_t s) {
    const size_t n = (size_t)M * W;
    if (n == 0 || !add.any()) return ZG_OK;
    add_two_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, add, n, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_tanh_norm(float* x, const float* pre, const float* nw, const int* rows, float* out, int n_rows, int W, hipStream_t s) {
    const size_t n = (size_t)n_rows * W;
    if (n == 0) return ZG_OK;
    ZG_REQUIRE((pre || nw) && (!nw || out) && !(pre && rows), ZG_ERR_ARG, "tanh norm: nothing to do, no output, or an in-place norm of gathered rows");
    const bool vec = W % 4 == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (vec) tanh_norm_kernel<4><<<(unsigned)((n / 4 + 255) / 256), 256, 0, s>>>(x, pre, nw, rows, out, n, W);
    else tanh_norm_kernel<1><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, pre, nw, rows, out, n, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_tanh_sum_norm(float* x, const SumParts& y, const float* nb, float mult, const float* nn, float* h, int M, int W, hipStream_t s) {
    const size_t n = (size_t)M * W;
    if (n == 0) return ZG_OK;
    ZG_REQUIRE(nb && (!nn || h) && (y.top == 0 || y.exp), ZG_ERR_ARG, "tanh norm behind a sum: no norm, no output, or no rows of the experts");
    const uintptr_t al = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(h) | reinterpret_cast<uintptr_t>(y.a) |
                         reinterpret_cast<uintptr_t>(y.exp) | reinterpret_cast<uintptr_t>(y.b);
    if (W % 4 == 0 && (al & 15) == 0) tanh_sum_norm_kernel<4><<<(unsigned)((n / 4 + 255) / 256), 256, 0, s>>>(x, y, nb, mult, nn, h, n, W);
    else tanh_sum_norm_kernel<1><<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, y, nb, mult, nn, h, n, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_plain(float* v, int ld, int rows_per_m, int width, int M, const float* w, float eps, hipStream_t s) {
    const int n_vec = M * rows_per_m;
    if (n_vec <= 0) return ZG_OK;
    norm_plain_kernel<<<(n_vec + 3) / 4, 256, 0, s>>>(v, ld, rows_per_m, width, n_vec, w, eps);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_hgrn2_scan(const float* proj, int ld, float* out, int ldo, float* state, size_t slot_stride, const int* ent_start,
                      const int* ent_len, const int* ent_slot, int n_entries, int M, int H, int D, int V, const float* bias, const float* low,
                      float* ws, size_t ws_floats, hipStream_t s, const float* decay, const GlaGate* gla) {
    if (n_entries <= 0) return ZG_OK;
    ZG_REQUIRE(!gla || (gla->z && gla->z_bias && !decay), ZG_ERR_ARG, "gated linear attention: its gate needs z and a bias, and no fixed decay");
    const GlaGate gg = gla ? *gla : GlaGate();
    ZG_REQUIRE(D >= 1 && D <= 16 * kScanRows, ZG_ERR_UNSUPPORTED, "hgrn2: %d key channels per head (at most %d)", D, 16 * kScanRows);
    if (decay && M > kGemvMaxRows && D <= 128 && ws && getenv("ZGPT2_LM_LINEAR_NO_CHUNKS") == nullptr) {
        // a scalar decay per head: chunks of kLinChunk tokens as matrix products (prompt portions; the test hook sends them through the scan)
        const int n_chunks = (M + kLinChunk - 1) / kLinChunk + n_entries;
        const size_t hf = (size_t)H * D * V;
        if (ws_floats >= (size_t)n_chunks * (hf + (size_t)H * D) && n_chunks <= 65535 && H <= 65535) {
            float* cB = ws;
            float* cA = ws + (size_t)n_chunks * hf;
            const dim3 grid(n_chunks, H);
            const int tiles = ((D + 31) / 32) * ((V + 31) / 32);
            linear_chunk_state_kernel<<<dim3(n_chunks, H, std::min(16, (tiles + 3) / 4)), 256, 0, s>>>(proj, ld, ent_start, ent_len, n_entries, H, D, V, decay, cB, cA);
            ZG_HIP(hipGetLastError());
            hgrn2_carry_kernel<<<dim3((unsigned)((hf + 255) / 256), n_entries), 256, 0, s>>>(state, slot_stride, ent_len, ent_slot, n_entries, H, D, V, cB,
                                                                                          cA, kLinChunk);
            ZG_HIP(hipGetLastError());
            const int dh = (D + 1) / 2;
            if (dh <= 8) linear_chunk_out_kernel<8><<<grid, 256, 0, s>>>(proj, ld, out, ldo, ent_start, ent_len, n_entries, H, D, V, decay, cB);
            else if (dh <= 16) linear_chunk_out_kernel<16><<<grid, 256, 0, s>>>(proj, ld, out, ldo, ent_start, ent_len, n_entries, H, D, V, decay, cB);
            else if (dh <= 32) linear_chunk_out_kernel<32><<<grid, 256, 0, s>>>(proj, ld, out, ldo, ent_start, ent_len, n_entries, H, D, V, decay, cB);
            else linear_chunk_out_kernel<64><<<grid, 256, 0, s>>>(proj, ld, out, ldo, ent_start, ent_len, n_entries, H, D, V, decay, cB);
            ZG_HIP(hipGetLastError());
            return ZG_OK;
        }
    }
    int G = 1;
    while (G * kScanRows < D) G <<= 1;
    const int Dp = G * kScanRows;
    int threads = ((V * G + 63) / 64) * 64;
    if (threads > 256) threads = 256;
    const int cols = threads / G;
    const int SB = std::max(1, std::min(kScanChunk, std::min((gla ? 2560 : 4096) / Dp, 8192 / cols)));
    const size_t lds = ((size_t)(gla ? 3 : 2) * SB * Dp + (size_t)SB * cols) * sizeof(float);
    // chunked when the step is long enough to pay for two passes, and the workspace holds every chunk's state
    const int max_chunks = (M + kScanChunk - 1) / kScanChunk + n_entries;
    const size_t head_floats = (size_t)H * D * V, need = (size_t)max_chunks * (head_floats + (size_t)H * D);
    const bool chunked = M >= 4 * kScanChunk && ws && ws_floats >= need;
    float* wsB = chunked ? ws : nullptr;
    float* wsA = chunked ? ws + (size_t)max_chunks * head_floats : nullptr;
#define ZG_SCAN_L(G_, KIND_, grid_x, mode)                                                                                                  \
    hgrn2_scan_kernel<G_, KIND_><<<dim3(grid_x, H, (V + cols - 1) / cols), threads, lds, s>>>(proj, ld, out, ldo, state, slot_stride, ent_start,    \
                                                                                               ent_len, ent_slot, n_entries, H, D, V, mode, SB, wsB, \
                                                                                               wsA, bias, low, decay, gg)
#define ZG_SCAN(G_, grid_x, mode)                         \
    do {                                                  \
        if (gla) ZG_SCAN_L(G_, SCAN_GLA, grid_x, mode);   \
        else if (decay) ZG_SCAN_L(G_, SCAN_LIN, grid_x, mode); \
        else ZG_SCAN_L(G_, SCAN_HGRN2, grid_x, mode);     \
    } while (0)
#define ZG_SCAN_G(grid_x, mode)                    \
    switch (G) {                                   \
        case 1: ZG_SCAN(1, grid_x, mode); break;   \
        case 2: ZG_SCAN(2, grid_x, mode); break;   \
        case 4: ZG_SCAN(4, grid_x, mode); break;   \
        case 8: ZG_SCAN(8, grid_x, mode); break;   \
        default: ZG_SCAN(16, grid_x, mode); break; \
    }
    if (!chunked) {
        ZG_SCAN_G(n_entries, SCAN_DIRECT);
        ZG_HIP(hipGetLastError());
        return ZG_OK;
    }
    ZG_SCAN_G(max_chunks, SCAN_A);
    ZG_HIP(hipGetLastError());
    hgrn2_carry_kernel<<<dim3((unsigned)((head_floats + 255) / 256), n_entries), 256, 0, s>>>(state, slot_stride, ent_len, ent_slot, n_entries, H, D, V,
                                                                                                wsB, wsA, kScanChunk);
    ZG_HIP(hipGetLastError());
    ZG_SCAN_G(max_chunks, SCAN_C);
    ZG_HIP(hipGetLastError());
#undef ZG_SCAN_G
#undef ZG_SCAN
#undef ZG_SCAN_L
    return ZG_OK;
}

int launch_latent_prep(const float* proj, int ld, int M, int q_rank, int KR, int R, const float* wq, const float* wkv, float eps, Rotary rot,
                       const int* row_pos, const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cq,
                       float* cache, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(rot.dims % 2 == 0 && rot.dims <= R, ZG_ERR_ARG, "rotary: %d rotated dimensions of a part of %d", rot.dims, R);
    latent_prep_kernel<<<M, 256, 0, s>>>(proj, ld, q_rank, KR, R, wq, wkv, eps, rot, row_pos, row_slot, page_table, max_pages, page_tokens, cq,
                                         cache);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_q_rotary(const float* q, int ldq, float* qa, int ldqa, int M, int H, int D, int R, int KR, Rotary rot, const int* row_pos,
                    hipStream_t s) {
    if (M <= 0 || R <= 0) return ZG_OK;
    q_rotary_kernel<<<M, 256, 0, s>>>(q, ldq, qa, ldqa, H, D, R, KR, rot, row_pos);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_latent_attention_tiles(const float* qa, float* ctx, int M, int H, int KR, int R, float scale, const int* ent_start, const int* ent_len,
                                  const int* ent_slot, int n_entries, const int* row_pos, const int* page_table, int max_pages, int page_tokens,
                                  const float* cache, hipStream_t s, bool* taken) {
    *taken = false;
    if (M <= 0 || n_entries <= 0) return ZG_OK;
    const int DT = KR + R;
    const dim3 grid((M + 31) / 32 + n_entries, (H + 3) / 4);
#define ZG_ATT_T(NKS_, NT_)                                                                                                                      \
    latent_attention_mfma_kernel<NKS_, NT_><<<grid, 256, 0, s>>>(qa, ctx, H, KR, R, scale, ent_start, ent_len, ent_slot, n_entries, row_pos, page_table, \
                                                                 max_pages, page_tokens, cache)
    if (DT <= 96 && KR <= 64) ZG_ATT_T(6, 2);
    else if (DT <= 160 && KR <= 128) ZG_ATT_T(10, 4);
    else if (DT <= 288 && KR <= 256) ZG_ATT_T(18, 8);
    else if (DT <= 384 && KR <= 320) ZG_ATT_T(24, 10);
    else return ZG_OK;  // larger latents: the caller's general kernel
#undef ZG_ATT_T
    ZG_HIP(hipGetLastError());
    *taken = true;
    return ZG_OK;
}

int launch_latent_attention(const float* qa, float* ctx, int M, int H, int KR, int R, float scale, const int* row_pos, const int* row_slot,
                            const int* page_table, int max_pages, int page_tokens, const float* cache, float* ws, size_t ws_floats,
                            hipStream_t s) {
    if (M <= 0) return ZG_OK;
    const int nd = (KR + R + 63) / 64;
    ZG_REQUIRE(nd <= 16, ZG_ERR_UNSUPPORTED, "latent attention: %d cached dimensions per token (at most 1024)", KR + R);
    // decode steps: the keys of a row in up to kAttnSplits ranges (a fixed grid, so that a captured step can be replayed at any
    // sequence length; ranges beyond the row's keys leave empty partials)
    int n_split = 1;
    if (M <= kGemvMaxRows && ws && ws_floats >= (size_t)M * H * kAttnSplits * (KR + 2) && (long long)max_pages * page_tokens > 128) n_split = kAttnSplits;
    const dim3 grid(M, H, n_split);
#define ZG_ATT(ND_)                                                                                                                           \
    latent_attention_kernel<ND_><<<grid, 256, 0, s>>>(qa, ctx, H, KR, R, scale, row_pos, row_slot, page_table, max_pages, page_tokens, cache, ws, \
                                                      n_split)
    if (nd <= 1) ZG_ATT(1);
    else if (nd <= 2) ZG_ATT(2);
    else if (nd <= 3) ZG_ATT(3);
    else if (nd <= 4) ZG_ATT(4);
    else if (nd <= 6) ZG_ATT(6);
    else if (nd <= 9) ZG_ATT(9);
    else if (nd <= 12) ZG_ATT(12);
    else ZG_ATT(16);
#undef ZG_ATT
    ZG_HIP(hipGetLastError());
    if (n_split > 1) {
        latent_merge_kernel<<<dim3(M, H), 256, 0, s>>>(ws, ctx, H, KR, n_split, row_pos);
        ZG_HIP(hipGetLastError());
    }
    return ZG_OK;
}

int launch_row_argmax(const float* logits, int rows, int n, float* max_out, int* idx_out, float* part_val, int* part_idx, hipStream_t s) {
    if (rows <= 0) return ZG_OK;
    const int parts = std::max(1, std::min(kArgmaxParts, (n + 1023) / 1024));
    row_argmax_kernel<<<dim3(rows, parts), 256, 0, s>>>(logits, n, nullptr, nullptr, part_val, part_idx, parts, 0);
    ZG_HIP(hipGetLastError());
    row_argmax_kernel<<<dim3(rows, 1), 256, 0, s>>>(logits, n, max_out, idx_out, part_val, part_idx, parts, 1);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

}  // namespace lm
}  // namespace zg
