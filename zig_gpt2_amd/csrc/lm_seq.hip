// lm_seq.hip — sequence mixers of the layered-model tier that carry more than a token shift from token to token:
//   * causal convolutions per channel whose last taps - 1 inputs live in a slot's state (the input convolution of a sublayer,
//     the short convolutions in front of the recurrences),
//   * softmax attention inside a sliding window over a paged cache of rotated keys and rotated VALUES, with a sink in the
//     denominator and the heads' weights mixed by a matrix; optionally the first tokens of a sequence stay visible behind the
//     window, and values may be cached unrotated,
//   * the real-gated linear recurrent unit (elementwise recurrence),
//   * the gated delta rule with one decay per key channel (a matrix state per head).
// Everything here is fp32 in both precision modes: positions, angles, scores, weights, gates, decays, recurrent states.
#include <math.h>
#include <stdlib.h>

#include <algorithm>

#include "lm_kernels.h"

namespace zg {
namespace lm {

namespace {

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

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

// ------------------------------------------------------------------------------------------------ embedding helpers
__global__ __launch_bounds__(256) void add_rows_kernel(float* x, const float* y, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += y[i];
}

// ------------------------------------------------------------------------------------------------ causal convolution
// Tap j of row m reads the input taps - 1 - j tokens back: a row of the same step when the entry brought that many tokens in
// front of m, else the slot's tail (the taps - 1 inputs before the step, oldest first; zeros for a new sequence).
constexpr int kMaxTaps = 16;
__global__ __launch_bounds__(256) void causal_conv_kernel(const float* in, int ld_in, float* out, int ld_out, int C, int taps, const float* w,
                                                          const float* bias, const float* pre_bias, int flags, float* tail, size_t slot_stride,
                                                          const int* row_off, const int* row_slot, int own_tail) {
    const int m = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int off = row_off[m], K = taps - 1;
    float* tl = tail + (size_t)row_slot[m] * slot_stride;
    const float pb = pre_bias ? pre_bias[c] : 0.0f;  // a bias of the input itself (the tail holds inputs with it)
    float acc = bias ? bias[c] : 0.0f;
    float val[kMaxTaps];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
        val[j] = 0.0f;
        if (j < taps) {
            const int src = off - K + j;
            val[j] = src >= 0 ? in[(size_t)(m - K + j) * ld_in + c] + pb : tl[(size_t)(K + src) * C + c];
            acc = fmaf(w[(size_t)c * taps + j], val[j], acc);
        }
    }
    if (flags & CONV_RESIDUAL) acc += in[(size_t)m * ld_in + c] + pb;
    if (flags & CONV_SILU) acc = silu_f(acc);
    out[(size_t)m * ld_out + c] = acc;
    if (own_tail) {  // the row is its entry's only one: this thread has read its channel's whole tail and moves it on itself
#pragma unroll
        for (int i = 0; i + 1 < kMaxTaps; ++i)
            if (i < K) tl[(size_t)i * C + c] = val[i + 1];
    }
}

// The new tail of every entry's slot: the last taps - 1 of (old tail, the entry's inputs).  A thread reads all it needs
// before it writes, and no other thread touches its channel of its slot.
__global__ __launch_bounds__(256) void conv_tail_kernel(const float* in, int ld_in, int C, int taps, const float* pre_bias, float* tail,
                                                        size_t slot_stride, const int* ent_start, const int* ent_len, const int* ent_slot) {
    const int e = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int n = ent_len[e], m0 = ent_start[e], K = taps - 1;
    if (n <= 0) return;
    float* tl = tail + (size_t)ent_slot[e] * slot_stride;
    const float pb = pre_bias ? pre_bias[c] : 0.0f;
    float val[kMaxTaps];
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
        if (i < K) {
            const int src = n - K + i;
            val[i] = src >= 0 ? in[(size_t)(m0 + src) * ld_in + c] + pb : tl[(size_t)(K + src) * C + c];
        }
#pragma unroll
    for (int i = 0; i < kMaxTaps; ++i)
        if (i < K) tl[(size_t)i * C + c] = val[i];
}

// Decode steps (one row per entry), rows of up to 256 * kSingleRegs floats held in registers: everything between two matrix
// products of a layer pass in one launch —
//   [x += x0]   or   [y = yl, or the mean of the two normed branches (yl / rms * wl + yr / rms * wr) / 2;  x += y / rms(y) * (1 + wb)]
//   h = x / rms(x) * (1 + wn);   out = h + conv(h) over the slot's tail;   the tail moved on by h.
constexpr int kSingleRegs = 8;
constexpr int kFastTaps = 4;
__global__ __launch_bounds__(256) void norm_conv_single_kernel(float* x, const float* x0, const float* yl, const float* yr, const float* wl,
                                                               const float* wr, const float* wb, const float* wn, float eps, int W, int taps,
                                                               const float* cw, float* tail, size_t slot_stride, const int* row_slot,
                                                               float* out) {
    __shared__ float s_red[8];
    const int m = blockIdx.x, K = taps - 1;
    float* xr = x + (size_t)m * W;
    float* tl = tail + (size_t)row_slot[m] * slot_stride;
    // every operand of the norms is requested before the first sum: one memory round trip
    float xv[kSingleRegs], yv[kSingleRegs], zv[kSingleRegs], wlv[kSingleRegs], wrv[kSingleRegs], wbv[kSingleRegs], wnv[kSingleRegs], t0v[kSingleRegs];
#pragma unroll
    for (int j = 0; j < kSingleRegs; ++j) {
        const int i = threadIdx.x + 256 * j;
        const bool ok = i < W;
        xv[j] = ok ? xr[i] + (x0 ? x0[(size_t)m * W + i] : 0.0f) : 0.0f;
        yv[j] = (ok && yl) ? yl[(size_t)m * W + i] : 0.0f;
        zv[j] = (ok && yr) ? yr[(size_t)m * W + i] : 0.0f;
        wlv[j] = (ok && yr) ? wl[i] : 0.0f;
        wrv[j] = (ok && yr) ? wr[i] : 0.0f;
        wbv[j] = (ok && yl) ? wb[i] : 0.0f;
        wnv[j] = ok ? wn[i] : 0.0f;
        t0v[j] = (ok && K > 0) ? tl[(size_t)(K - 1) * W + i] : 0.0f;  // the newest tail entry
    }
    // convolutions of up to kFastTaps taps: their weights and the whole tail travel in the same round trip
    float cwv[kSingleRegs][kFastTaps], tlv[kSingleRegs][kFastTaps - 1];
    const bool fast = taps <= kFastTaps;
    if (fast) {
#pragma unroll
        for (int j = 0; j < kSingleRegs; ++j) {
            const int i = threadIdx.x + 256 * j;
#pragma unroll
            for (int t = 0; t < kFastTaps; ++t) cwv[j][t] = (i < W && t < taps) ? cw[(size_t)i * taps + t] : 0.0f;
#pragma unroll
            for (int t = 0; t < kFastTaps - 1; ++t) tlv[j][t] = (i < W && t < K) ? tl[(size_t)t * W + i] : 0.0f;
        }
    }
    if (yl) {
        if (yr) {
            float sa = 0.0f, sb = 0.0f;
#pragma unroll
            for (int j = 0; j < kSingleRegs; ++j) {
                sa = fmaf(yv[j], yv[j], sa);
                sb = fmaf(zv[j], zv[j], sb);
            }
            sa = block_allsum(sa, s_red);
            sb = block_allsum(sb, s_red);
            const float ra = 1.0f / sqrtf(sa / (float)W + eps), rb = 1.0f / sqrtf(sb / (float)W + eps);
#pragma unroll
            for (int j = 0; j < kSingleRegs; ++j) yv[j] = 0.5f * (yv[j] * ra * wlv[j] + zv[j] * rb * wrv[j]);
        }
        float sy = 0.0f;
#pragma unroll
        for (int j = 0; j < kSingleRegs; ++j) sy = fmaf(yv[j], yv[j], sy);
        sy = block_allsum(sy, s_red);
        const float ry = 1.0f / sqrtf(sy / (float)W + eps);
#pragma unroll
        for (int j = 0; j < kSingleRegs; ++j) xv[j] += yv[j] * ry * (1.0f + wbv[j]);
    }
    float sx = 0.0f;
#pragma unroll
    for (int j = 0; j < kSingleRegs; ++j) sx = fmaf(xv[j], xv[j], sx);
    sx = block_allsum(sx, s_red);
    const float rx = 1.0f / sqrtf(sx / (float)W + eps);
#pragma unroll
    for (int j = 0; j < kSingleRegs; ++j) {
        const int i = threadIdx.x + 256 * j;
        if (i < W) {
            if (x0 || yl) xr[i] = xv[j];
            const float h = xv[j] * rx * (1.0f + wnv[j]);
            if (fast) {
                float acc = 0.0f;
#pragma unroll
                for (int t = 0; t < kFastTaps; ++t) acc = fmaf(cwv[j][t], t == K ? h : t < kFastTaps - 1 ? tlv[j][t] : 0.0f, acc);
#pragma unroll
                for (int t = 1; t < kFastTaps - 1; ++t)
                    if (t < K) tl[(size_t)(t - 1) * W + i] = tlv[j][t];
                if (K > 0) tl[(size_t)(K - 1) * W + i] = h;
                out[(size_t)m * W + i] = h + acc;
                continue;
            }
            float acc = cw[(size_t)i * taps + K] * h;
            for (int t = 0; t < K; ++t) {  // tail entry t is taps - 1 - t tokens back; it moves one place towards the front
                const float tv = t == K - 1 ? t0v[j] : tl[(size_t)t * W + i];
                acc = fmaf(cw[(size_t)i * taps + t], tv, acc);
                if (t > 0) tl[(size_t)(t - 1) * W + i] = tv;
            }
            if (K > 0) tl[(size_t)(K - 1) * W + i] = h;
            out[(size_t)m * W + i] = h + acc;
        }
    }
}

// ------------------------------------------------------------------------------------------------ windowed attention
// proj rows: [q (H D) | k (G D) | v (G V)].  q is rotated in place (pairs (2i, 2i + 1) below rot.dims); the rotated key and the
// value rotated over ALL its channels (pair i by pos * vfreq[i]) go to the token's cache row [G D | G V].
__global__ __launch_bounds__(256) void window_prep_kernel(float* proj, int ld, int H, int G, int D, int V, Rotary rot, const float* vfreq,
                                                          const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                          int page_tokens, float* cache) {
    const int m = blockIdx.x;
    const int pos = row_pos[m];
    const int page = page_table[(size_t)row_slot[m] * max_pages + (pos / page_tokens) % max_pages];
    float* crow = cache + ((size_t)page * page_tokens + pos % page_tokens) * ((size_t)G * (D + V));
    float* row = proj + (size_t)m * ld;
    const float fpos = (float)pos;
    const int half = rot.dims / 2;
    for (int idx = threadIdx.x; idx < H * half; idx += blockDim.x) {
        const int h = idx / half, i = idx % half;
        float* p = row + (size_t)h * D + 2 * i;
        float sn, cs;
        sincosf(fpos * rot.freq[i], &sn, &cs);
        const float a = p[0], b = p[1];
        p[0] = (a * cs - b * sn) * rot.amp;
        p[1] = (b * cs + a * sn) * rot.amp;
    }
    const float* k = row + (size_t)H * D;
    for (int idx = threadIdx.x; idx < G * D; idx += blockDim.x) {
        const int i = idx % D;
        float out;
        if (i < rot.dims) {
            float sn, cs;
            sincosf(fpos * rot.freq[i >> 1], &sn, &cs);
            const float own = k[idx], other = k[idx - i + (i ^ 1)];
            out = ((i & 1) ? own * cs + other * sn : own * cs - other * sn) * rot.amp;
        } else {
            out = k[idx];
        }
        crow[idx] = out;
    }
    const float* v = k + (size_t)G * D;
    for (int idx = threadIdx.x; idx < G * V; idx += blockDim.x) {
        const int i = idx % V;
        float sn, cs;
        sincosf(fpos * vfreq[i >> 1], &sn, &cs);
        const float own = v[idx], other = v[idx - i + (i ^ 1)];
        crow[(size_t)G * D + idx] = (i & 1) ? own * cs + other * sn : own * cs - other * sn;
    }
}

// One workgroup per query row, all heads together (the mix of the heads' weights needs every head's weight of a key).
// Keys are walked in tiles of kWinTile, twice: first the per-head maximum and denominator (with exp(sink) in it), then the
// normalised weights, their mix over the heads, and the weighted sum of the values of the head's own key/value head.  The
// result is turned back by the query's position and stored.  Tiles start at the first key of the window: the order of every
// sum depends on the position alone.
// The keys a row sees, numbered from 0: first the kept tokens that lie in front of its window (the first `keep` positions of the
// sequence stay visible), then the window's keys up to the row's own position.  Every kernel below walks this numbering, so the
// order of a row's sums depends on its position alone.
struct KeySpan {
    int j_lo, n_first, n_keys;
};
__device__ __forceinline__ KeySpan key_span(int pos, int window, int keep) {
    KeySpan k;
    k.j_lo = window > 0 ? max(0, pos - window + 1) : 0;
    k.n_first = min(keep, k.j_lo);
    k.n_keys = k.n_first + pos - k.j_lo + 1;
    return k;
}
__device__ __forceinline__ int key_pos(const KeySpan& k, int n) { return n < k.n_first ? n : k.j_lo + (n - k.n_first); }

// a scaled score on its way to the softmax: capped, then less the head's slope per position of distance (fp32)
__device__ __forceinline__ float shape_score(float sc, const ScoreShape& sh, int h, int dist) {
    if (sh.cap > 0.0f) sc = sh.cap * tanhf(sc / sh.cap);
    if (sh.slope) sc -= sh.slope[h] * (float)dist;
    return sc;
}

constexpr int kWinTile = 64;
constexpr int kWinMaxHeads = 64;
constexpr int kWinAcc = 16;  // outputs per thread: H * V <= 256 * kWinAcc

__global__ __launch_bounds__(256) void window_attention_kernel(const float* q, int ldq, float* out, int ldo, int H, int G, int D, int V,
                                                               float scale, int window, int keep, const float* sink, const float* talk,
                                                               const float* vfreq, const int* row_pos, const int* row_slot,
                                                               const int* page_table, int max_pages, int page_tokens, const float* cache,
                                                               const ScoreShape shape) {
    extern __shared__ __attribute__((aligned(16))) float s_win[];
    float* s_q = s_win;                       // [H D]
    float* s_s = s_q + H * D;                 // [H][kWinTile] scores, then weights
    float* s_w = s_s + H * kWinTile;          // [H][kWinTile] mixed weights
    float* s_talk = s_w + H * kWinTile;       // [H H]
    float* s_o = s_talk + H * H;              // [H V]
    __shared__ float s_max[kWinMaxHeads], s_den[kWinMaxHeads];
    __shared__ int s_row[kWinTile];  // cache row of every key of the tile
    const int m = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pos = row_pos[m];
    const int* pages = page_table + (size_t)row_slot[m] * max_pages;
    const KeySpan span = key_span(pos, window, keep);
    const int n_keys = span.n_keys;
    const int rep = H / G;
    const size_t cstride = (size_t)G * (D + V);
    for (int i = tid; i < H * D; i += blockDim.x) s_q[i] = q[(size_t)m * ldq + i];
    for (int i = tid; i < H * H; i += blockDim.x) s_talk[i] = talk ? talk[i] : ((i / H) == (i % H) ? 1.0f : 0.0f);
    if (tid < H) {
        s_max[tid] = sink ? sink[tid] : -INFINITY;
        s_den[tid] = sink ? 1.0f : 0.0f;
    }
    float acc[kWinAcc];
#pragma unroll
    for (int r = 0; r < kWinAcc; ++r) acc[r] = 0.0f;

    auto tile_scores = [&](int t0, int nt) {
        __syncthreads();
        if (tid < nt) {
            const int j = key_pos(span, t0 + tid);
            s_row[tid] = pages[(j / page_tokens) % max_pages] * page_tokens + j % page_tokens;
        }
        __syncthreads();
        for (int idx = tid; idx < H * kWinTile; idx += blockDim.x) {
            const int h = idx / kWinTile, jj = idx % kWinTile;
            float s = -INFINITY;
            if (jj < nt) {
                const float* kr = cache + (size_t)s_row[jj] * cstride + (size_t)(h / rep) * D;
                const float* qh = s_q + h * D;
                float a = 0.0f;
                for (int d = 0; d < D; ++d) a = fmaf(qh[d], kr[d], a);
                s = shape_score(a * scale, shape, h, pos - key_pos(span, t0 + jj));
            }
            s_s[idx] = s;
        }
        __syncthreads();
    };

    for (int t0 = 0; t0 < n_keys; t0 += kWinTile) {  // pass 1: maximum and denominator per head
        const int nt = min(kWinTile, n_keys - t0);
        tile_scores(t0, nt);
        for (int h = wave; h < H; h += 4) {
            const float s = s_s[h * kWinTile + lane];
            const float mo = s_max[h], mn = fmaxf(mo, wave_allmax(s));
            const float part = wave_allsum(lane < nt ? expf(s - mn) : 0.0f);
            if (lane == 0) {
                s_den[h] = s_den[h] * expf(mo - mn) + part;
                s_max[h] = mn;
            }
        }
    }
    for (int t0 = 0; t0 < n_keys; t0 += kWinTile) {  // pass 2: weights, their mix, values
        const int nt = min(kWinTile, n_keys - t0);
        tile_scores(t0, nt);
        for (int idx = tid; idx < H * kWinTile; idx += blockDim.x) {
            const int h = idx / kWinTile, jj = idx % kWinTile;
            s_s[idx] = jj < nt ? expf(s_s[idx] - s_max[h]) / s_den[h] : 0.0f;
        }
        __syncthreads();
        for (int idx = tid; idx < H * kWinTile; idx += blockDim.x) {
            const int h = idx / kWinTile, jj = idx % kWinTile;
            float wsum = 0.0f;
            for (int g = 0; g < H; ++g) wsum = fmaf(s_talk[h * H + g], s_s[g * kWinTile + jj], wsum);
            s_w[idx] = wsum;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kWinAcc; ++r) {
            const int o = tid + 256 * r;
            if (o < H * V) {
                const int h = o / V, c = o % V;
                const float* vbase = cache + (size_t)G * D + (size_t)(h / rep) * V + c;
                float a = acc[r];
                for (int jj = 0; jj < nt; ++jj) a = fmaf(s_w[h * kWinTile + jj], vbase[(size_t)s_row[jj] * cstride], a);
                acc[r] = a;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kWinAcc; ++r) {
        const int o = tid + 256 * r;
        if (o < H * V) s_o[o] = acc[r];
    }
    __syncthreads();
    const float fpos = (float)pos;
    for (int o = tid; o < H * V; o += blockDim.x) {  // turned back by the query's position
        const int i = o % V;
        if (!vfreq) {
            out[(size_t)m * ldo + o] = s_o[o];
            continue;
        }
        float sn, cs;
        sincosf(fpos * vfreq[i >> 1], &sn, &cs);
        const float own = s_o[o], other = s_o[o - i + (i ^ 1)];
        out[(size_t)m * ldo + o] = (i & 1) ? own * cs - other * sn : own * cs + other * sn;
    }
}

// The same attention with a row's keys split over several workgroups, in three launches (scores and weights pass through a
// workspace, so no score is computed twice and a one-row step still fills many compute units):
//   scores   workgroup (split, row): s_h(j) for its share of the row's keys — a wave per key, lanes over the D channels, one
//            wave reduction per head — written to sc[row][h][j - first key]; per head the share's maximum and sum of exp
//   mix      workgroup (split, row): the row's maximum and denominator per head from all shares (and the sink), then for its
//            keys the normalised weights, their mix over the heads, and the share's weighted sum of values
//   merge    workgroup (row): the shares' sums added in split order, turned back by the row's position
// A share is ceil(keys of the row / splits) consecutive keys: the order of every sum depends on the position alone.
constexpr int kMixTile = 32;

__device__ __forceinline__ KeySpan window_range(int pos, int window, int keep, int n_split, int split, int& k0, int& k1) {
    const KeySpan span = key_span(pos, window, keep);
    const int chunk = (span.n_keys + n_split - 1) / n_split;
    k0 = min(span.n_keys, split * chunk);
    k1 = min(span.n_keys, k0 + chunk);
    return span;
}

constexpr int kScoreTile = 128;  // keys whose scores a workgroup holds in the LDS at a time
constexpr int kScoreKeys = 8;    // keys a wave has in flight

template <int RPL>
__global__ __launch_bounds__(256) void window_scores_kernel(const float* q, int ldq, int H, int G, int D, int V, float scale, int window,
                                                            int keep, const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                            int page_tokens, const float* cache, float* sc, int NK, float* st,
                                                            const ScoreShape shape) {
    extern __shared__ __attribute__((aligned(16))) float s_sc[];
    float* s_q = s_sc;                     // [H][64 RPL] (zero beyond D)
    float* s_t = s_q + H * 64 * RPL;       // [H][kScoreTile] scores of the tile
    float* s_m = s_t + H * kScoreTile;     // [H] running maximum
    float* s_l = s_m + H;                  // [H] running sum of exp
    __shared__ int s_row[kScoreTile];
    const int split = blockIdx.x, n_split = gridDim.x, m = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pos = row_pos[m];
    int k0, k1;
    const KeySpan span = window_range(pos, window, keep, n_split, split, k0, k1);
    const int* pages = page_table + (size_t)row_slot[m] * max_pages;
    const int rep = H / G;
    const size_t cstride = (size_t)G * (D + V);
    for (int i = threadIdx.x; i < H * 64 * RPL; i += blockDim.x) {
        const int h = i / (64 * RPL), d = i % (64 * RPL);
        s_q[i] = d < D ? q[(size_t)m * ldq + (size_t)h * D + d] : 0.0f;
    }
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        s_m[i] = -INFINITY;
        s_l[i] = 0.0f;
    }
    float* srow = sc + (size_t)m * H * NK;
    for (int t0 = k0; t0 < k1; t0 += kScoreTile) {
        const int nt = min(kScoreTile, k1 - t0);
        __syncthreads();  // the tile before has been consumed (and, the first time, q is staged)
        for (int i = threadIdx.x; i < nt; i += blockDim.x) {
            const int j = key_pos(span, t0 + i);
            s_row[i] = pages[(j / page_tokens) % max_pages] * page_tokens + j % page_tokens;
        }
        __syncthreads();
        // a wave takes kScoreKeys keys at a time: all their loads are requested before the first product
        for (int kk = wave * kScoreKeys; kk < nt; kk += 4 * kScoreKeys) {
            for (int g = 0; g < G; ++g) {
                float kd[kScoreKeys][RPL];
#pragma unroll
                for (int u = 0; u < kScoreKeys; ++u) {
                    const float* kr = cache + (size_t)s_row[min(kk + u, nt - 1)] * cstride + (size_t)g * D;
#pragma unroll
                    for (int r = 0; r < RPL; ++r) kd[u][r] = lane + 64 * r < D ? kr[lane + 64 * r] : 0.0f;
                }
                for (int hh = 0; hh < rep; ++hh) {
                    const int h = g * rep + hh;
                    float a[kScoreKeys];
#pragma unroll
                    for (int u = 0; u < kScoreKeys; ++u) {
                        a[u] = 0.0f;
#pragma unroll
                        for (int r = 0; r < RPL; ++r) a[u] = fmaf(s_q[h * 64 * RPL + lane + 64 * r], kd[u][r], a[u]);
                    }
#pragma unroll
                    for (int u = 0; u < kScoreKeys; ++u) a[u] = wave_allsum(a[u]) * scale;
                    if (lane < kScoreKeys && kk + lane < nt) {
                        float mine = a[0];
#pragma unroll
                        for (int u = 1; u < kScoreKeys; ++u) mine = lane == u ? a[u] : mine;
                        mine = shape_score(mine, shape, h, pos - key_pos(span, t0 + kk + lane));
                        s_t[h * kScoreTile + kk + lane] = mine;
                        srow[(size_t)h * NK + t0 + kk + lane] = mine;
                    }
                }
            }
        }
        __syncthreads();
        for (int h = wave; h < H; h += 4) {  // the tile's share of the head's maximum and sum, a wave per head
            float mx = -INFINITY;
            for (int i = lane; i < nt; i += 64) mx = fmaxf(mx, s_t[h * kScoreTile + i]);
            mx = fmaxf(wave_allmax(mx), s_m[h]);
            float l = 0.0f;
            for (int i = lane; i < nt; i += 64) l += expf(s_t[h * kScoreTile + i] - mx);
            l = wave_allsum(l);
            if (lane == 0) {
                s_l[h] = (s_l[h] > 0.0f ? s_l[h] * expf(s_m[h] - mx) : 0.0f) + l;
                s_m[h] = mx;
            }
        }
    }
    __syncthreads();
    for (int h = threadIdx.x; h < H; h += blockDim.x) {
        float* o = st + (((size_t)m * n_split + split) * H + h) * 2;
        o[0] = s_m[h];
        o[1] = s_l[h];
    }
}

// Prompt portions: the scores of 32 consecutive rows of an entry against tiles of 32 keys on the matrix cores, in true fp32
// (v_mfma_f32_32x32x2_f32 in both precision modes): a key is read once per 32 rows instead of once per row, and no score needs a
// cross-lane reduction.  Lane (r, half) of a wave holds the channels half * Dh .. + Dh of query row r and of key r (the order of
// the channels inside the sum is free), so both operands are contiguous runs of a row.  A wave takes (key tile, key head) units;
// the row's statistics follow in window_stats_kernel.
typedef __attribute__((ext_vector_type(16))) float f32x16_t;

__device__ __forceinline__ bool rows_find_block(int id, const int* ent_len, int n_entries, int& e, int& b) {
    for (e = 0; e < n_entries; ++e) {
        const int nb = (ent_len[e] + 31) / 32;
        if (id < nb) {
            b = id;
            return true;
        }
        id -= nb;
    }
    return false;
}

template <int DH>
__global__ __launch_bounds__(256) void window_scores_mfma_kernel(const float* q, int ldq, int H, int G, int D, int V, float scale, int window,
                                                                 int keep, const int* ent_start, const int* ent_len, int n_entries, const int* row_pos,
                                                                 const int* row_slot, const int* page_table, int max_pages, int page_tokens,
                                                                 const float* cache, float* sc, int NK, const ScoreShape shape) {
    int e, b;
    if (!rows_find_block(blockIdx.x, ent_len, n_entries, e, b)) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 31, kh = lane >> 5;
    const int m0 = ent_start[e] + 32 * b, nrows = min(32, ent_len[e] - 32 * b);
    const int pos0 = row_pos[m0], pos_last = pos0 + nrows - 1;
    // the block's keys, numbered like a row's: the kept tokens in front of the FIRST row's window, then everything from there to
    // the last row's position (a superset of every row's keys; each pair is masked by its own row's span below)
    const KeySpan blk = key_span(pos0, window, keep);
    const int n_blk = blk.n_first + pos_last - blk.j_lo + 1;
    const int n_tiles = (n_blk - 1) / 32 + 1, units = n_tiles * G;
    const int* pages = page_table + (size_t)row_slot[m0] * max_pages;
    const int rep = H / G, Dh = (D + 1) / 2;
    const size_t cstride = (size_t)G * (D + V);
    const bool vec = D % 8 == 0 && V % 4 == 0 && ldq % 4 == 0 && ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(cache)) & 15) == 0;
    for (int u = blockIdx.y * 4 + wave; u < units; u += 4 * gridDim.y) {
        const int tile = u / G, g = u % G;
        const int nk = 32 * tile + r;                          // the key's number inside the block
        const int j = nk < n_blk ? key_pos(blk, nk) : pos_last + 1;  // its position (beyond the block: none)
        float kreg[DH];
        {
            const int jc = min(j, pos_last);
            const float* kr = cache + ((size_t)pages[(jc / page_tokens) % max_pages] * page_tokens + jc % page_tokens) * cstride + (size_t)g * D + kh * Dh;
            if (vec) {  // 16-byte loads: a lane's run of channels starts on a 16-byte boundary and is a multiple of four long
#pragma unroll
                for (int t = 0; t < DH; t += 4) {
                    const f32x4 x = (j <= pos_last && t < Dh) ? *reinterpret_cast<const f32x4*>(kr + t) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    kreg[t] = x.x; kreg[t + 1] = x.y; kreg[t + 2] = x.z; kreg[t + 3] = x.w;
                }
            } else {
#pragma unroll
                for (int t = 0; t < DH; ++t) kreg[t] = (j <= pos_last && t < Dh && kh * Dh + t < D) ? kr[t] : 0.0f;
            }
        }
        for (int hh = 0; hh < rep; ++hh) {
            const int h = g * rep + hh;
            const float* qr = q + (size_t)(m0 + min(r, nrows - 1)) * ldq + (size_t)h * D + kh * Dh;
            float qreg[DH];
            if (vec) {
#pragma unroll
                for (int t = 0; t < DH; t += 4) {
                    const f32x4 x = (r < nrows && t < Dh) ? *reinterpret_cast<const f32x4*>(qr + t) : f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                    qreg[t] = x.x; qreg[t + 1] = x.y; qreg[t + 2] = x.z; qreg[t + 3] = x.w;
                }
            } else {
#pragma unroll
                for (int t = 0; t < DH; ++t) qreg[t] = (r < nrows && t < Dh && kh * Dh + t < D) ? qr[t] : 0.0f;
            }
            f32x16_t acc;
#pragma unroll
            for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
            for (int t = 0; t < DH; ++t) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qreg[t], kreg[t], acc, 0, 0, 0);
            // accumulator element i: query row 8 (i / 4) + 4 half + i % 4 of the block, key r of the tile
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int qi = 8 * (i >> 2) + 4 * kh + (i & 3);
                const int pi = pos0 + qi;
                const KeySpan sp = key_span(pi, window, keep);
                if (qi < nrows && j <= pi && (j >= sp.j_lo || j < sp.n_first))
                    sc[((size_t)(m0 + qi) * H + h) * NK + (j >= sp.j_lo ? sp.n_first + (j - sp.j_lo) : j)] = shape_score(acc[i] * scale, shape, h, pi - j);
            }
        }
    }
}

// Per row and head the maximum and the sum of exp of the row's scores (a wave per head, its lanes over the keys), filed as the
// statistics of share 0; the other shares are marked empty.
__global__ __launch_bounds__(256) void window_stats_kernel(const float* sc, int NK, int H, int window, int keep, int n_split, const int* row_pos,
                                                           float* st) {
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pos = row_pos[m];
    const int n_keys = key_span(pos, window, keep).n_keys;
    for (int h = wave; h < H; h += 4) {
        const float* sr = sc + ((size_t)m * H + h) * NK;
        float mx = -INFINITY;
        for (int i = lane; i < n_keys; i += 64) mx = fmaxf(mx, sr[i]);
        mx = wave_allmax(mx);
        float l = 0.0f;
        for (int i = lane; i < n_keys; i += 64) l += expf(sr[i] - mx);
        l = wave_allsum(l);
        for (int s2 = lane; s2 < n_split; s2 += 64) {
            float* o = st + (((size_t)m * n_split + s2) * H + h) * 2;
            o[0] = s2 == 0 ? mx : -INFINITY;
            o[1] = s2 == 0 ? l : 0.0f;
        }
    }
}

__global__ __launch_bounds__(256) void window_mix_kernel(int H, int G, int D, int V, int window, int keep, const float* sink, const float* talk,
                                                         const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                         int page_tokens, const float* cache, const float* sc, int NK, const float* st,
                                                         float* po) {
    extern __shared__ __attribute__((aligned(16))) float s_mx[];
    float* s_p = s_mx;                  // [H][kMixTile]
    float* s_w = s_p + H * kMixTile;    // [H][kMixTile]
    float* s_talk = s_w + H * kMixTile; // [H H]
    float* s_M = s_talk + H * H;        // [H]
    float* s_iZ = s_M + H;              // [H]
    __shared__ int s_row[kMixTile];
    const int split = blockIdx.x, n_split = gridDim.x, m = blockIdx.y, tid = threadIdx.x;
    const int pos = row_pos[m];
    int k0, k1;
    const KeySpan span = window_range(pos, window, keep, n_split, split, k0, k1);
    const int* pages = page_table + (size_t)row_slot[m] * max_pages;
    const int rep = H / G;
    const size_t cstride = (size_t)G * (D + V);
    for (int i = tid; i < H * H; i += blockDim.x) s_talk[i] = talk ? talk[i] : ((i / H) == (i % H) ? 1.0f : 0.0f);
    for (int h = tid >> 6; h < H; h += 4) {  // a wave per head, its lanes over the shares (at most kWinSplits = 64): one round trip
        const int lane = tid & 63;
        const float* sp = st + (((size_t)m * n_split + lane) * H + h) * 2;
        const float pm = lane < n_split ? sp[0] : -INFINITY, pl = lane < n_split ? sp[1] : 0.0f;
        const float sk = sink ? sink[h] : -INFINITY;
        const float mx = fmaxf(wave_allmax(pm), sk);
        const float z = wave_allsum(pl > 0.0f ? pl * expf(pm - mx) : 0.0f) + (sink ? expf(sk - mx) : 0.0f);
        if (lane == 0) {
            s_M[h] = mx;
            s_iZ[h] = 1.0f / z;
        }
    }
    float acc[kWinAcc];
#pragma unroll
    for (int r = 0; r < kWinAcc; ++r) acc[r] = 0.0f;
    const float* srow = sc + (size_t)m * H * NK;
    for (int t0 = k0; t0 < k1; t0 += kMixTile) {
        const int nt = min(kMixTile, k1 - t0);
        __syncthreads();
        if (tid < nt) {
            const int j = key_pos(span, t0 + tid);
            s_row[tid] = pages[(j / page_tokens) % max_pages] * page_tokens + j % page_tokens;
        }
        for (int idx = tid; idx < H * kMixTile; idx += blockDim.x) {
            const int h = idx / kMixTile, jj = idx % kMixTile;
            s_p[idx] = jj < nt ? expf(srow[(size_t)h * NK + t0 + jj] - s_M[h]) * s_iZ[h] : 0.0f;
        }
        __syncthreads();
        for (int idx = tid; idx < H * kMixTile; idx += blockDim.x) {
            const int h = idx / kMixTile, jj = idx % kMixTile;
            float wsum = s_p[idx];  // no mixing matrix: every head keeps its own weights
            if (talk) {
                wsum = 0.0f;
                for (int g = 0; g < H; ++g) wsum = fmaf(s_talk[h * H + g], s_p[g * kMixTile + jj], wsum);
            }
            s_w[idx] = wsum;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kWinAcc; ++r) {
            const int o = tid + 256 * r;
            if (o < H * V) {
                const int h = o / V, c = o % V;
                const float* vbase = cache + (size_t)G * D + (size_t)(h / rep) * V + c;
                float a = acc[r];
                for (int j0 = 0; j0 < nt; j0 += 8) {  // eight values requested together (keys beyond the tile weigh nothing)
                    float vv[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) vv[u] = vbase[(size_t)s_row[min(j0 + u, nt - 1)] * cstride];
#pragma unroll
                    for (int u = 0; u < 8; ++u) a = fmaf(s_w[h * kMixTile + j0 + u], vv[u], a);
                }
                acc[r] = a;
            }
        }
    }
    float* orow = po + ((size_t)m * n_split + split) * H * V;
#pragma unroll
    for (int r = 0; r < kWinAcc; ++r) {
        const int o = tid + 256 * r;
        if (o < H * V) orow[o] = acc[r];
    }
}

// Prompt portions: normalised weights, their mix over the heads and the weighted value sums for 32 consecutive rows of an entry,
// the value product on the matrix cores in true fp32.  Per tile of kPvKeys keys: every thread takes (row, key) pairs — the
// weights of all heads from the scores and the rows' statistics (with the sink), mixed in registers, written to the LDS as
// [head][row][key]; then a wave owns (head, 32 value channels) units whose accumulators live across the tiles: A = the mixed
// weights of its head (row x key), B = the values of the head's key head (channel x key, read once per 32 rows).  Shares of
// the block's key range go to blockIdx.y (the merge adds them), groups of kPvUnits * 4 units to blockIdx.z.
constexpr int kPvKeys = 16;
constexpr int kPvUnits = 3;  // (head, channel tile) units a wave accumulates (few: two workgroups share a compute unit and hide each other's loads)
constexpr int kPvHeads = 16; // most heads a workgroup weighs (a pair's weights of these heads sit in registers)
// Without a mixing matrix the heads are independent: a workgroup then weighs only the heads of its own units (at most
// pv_block_heads of them), so any number of heads fits and no score is read by more than one group of units.
__host__ __device__ constexpr int pv_block_heads(int ctiles) { return (4 * kPvUnits - 1) / ctiles + 2; }

__global__ __launch_bounds__(256) void window_mix_mfma_kernel(int H, int G, int D, int V, int window, int keep, const float* sink, const float* talk,
                                                              const int* ent_start, const int* ent_len, int n_entries, const int* row_pos,
                                                              const int* row_slot, const int* page_table, int max_pages, int page_tokens,
                                                              const float* cache, const float* sc, int NK, const float* st, int n_split,
                                                              float* po) {
    extern __shared__ __attribute__((aligned(16))) float s_pv[];
    constexpr int KP = kPvKeys + 1;           // padded key stride
    const int ctiles = (V + 31) / 32, units = H * ctiles;
    // the heads this workgroup weighs: all of them under a mixing matrix, else those of its own units
    const int ub0 = blockIdx.z * 4 * kPvUnits;
    const int h_lo = talk ? 0 : min(H - 1, ub0 / ctiles);
    const int h_n = talk ? H : min(H, (ub0 + 4 * kPvUnits - 1) / ctiles + 1) - h_lo;
    const int hs = talk ? H : min(H, pv_block_heads(ctiles));
    float* s_w = s_pv;                        // [hs][32][KP] mixed weights of the tile (head h at h - h_lo)
    float* s_talk = s_w + hs * 32 * KP;       // [H H]
    float* s_M = s_talk + H * H;              // [32][H]
    float* s_iZ = s_M + 32 * H;               // [32][H]
    __shared__ int s_row[kPvKeys];
    int e, b;
    if (!rows_find_block(blockIdx.x, ent_len, n_entries, e, b)) return;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 31, kh = lane >> 5;
    const int m0 = ent_start[e] + 32 * b, nrows = min(32, ent_len[e] - 32 * b);
    const int pos0 = row_pos[m0], pos_last = pos0 + nrows - 1;
    const KeySpan blk = key_span(pos0, window, keep);  // the block's keys, numbered as in window_scores_mfma_kernel
    const int n_blk = blk.n_first + pos_last - blk.j_lo + 1;
    const int n_tiles = (n_blk - 1) / kPvKeys + 1, per = (n_tiles + gridDim.y - 1) / gridDim.y;
    const int t_lo = min(n_tiles, (int)blockIdx.y * per), t_hi = min(n_tiles, t_lo + per);
    const int* pages = page_table + (size_t)row_slot[m0] * max_pages;
    const int rep = H / G;
    const size_t cstride = (size_t)G * (D + V);
    if (talk)
        for (int i = tid; i < H * H; i += blockDim.x) s_talk[i] = talk[i];
    for (int i = tid; i < 32 * H; i += blockDim.x) {  // the rows' maximum and denominator per head, the sink counted once
        const int row = i / H, h = i % H;
        float mx = 0.0f, iz = 0.0f;
        if (row < nrows) {
            const float* sp = st + (((size_t)(m0 + row) * n_split) * H + h) * 2;
            const float sk = sink ? sink[h] : -INFINITY;
            mx = fmaxf(sp[0], sk);
            iz = 1.0f / (sp[1] * expf(sp[0] - mx) + (sink ? expf(sk - mx) : 0.0f));
        }
        s_M[i] = mx;
        s_iZ[i] = iz;
    }
    f32x16_t acc[kPvUnits];
#pragma unroll
    for (int u = 0; u < kPvUnits; ++u)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[u][i] = 0.0f;
    const int u0 = (blockIdx.z * 4 + wave) * kPvUnits;  // this wave's first unit
    for (int tile = t_lo; tile < t_hi; ++tile) {
        const int n0 = kPvKeys * tile;
        __syncthreads();  // the tile before has been consumed (and, the first time, the statistics are staged)
        if (tid < kPvKeys) {
            const int jc = n0 + tid < n_blk ? key_pos(blk, n0 + tid) : pos_last;
            s_row[tid] = pages[(jc / page_tokens) % max_pages] * page_tokens + jc % page_tokens;
        }
        for (int pr = tid; pr < 32 * kPvKeys; pr += blockDim.x) {
            const int row = pr / kPvKeys, kk = pr % kPvKeys, pi = pos0 + row;
            const int j = n0 + kk < n_blk ? key_pos(blk, n0 + kk) : pos_last + 1;
            const KeySpan sp = key_span(pi, window, keep);
            const bool ok = row < nrows && j <= pi && (j >= sp.j_lo || j < sp.n_first);
            float p[kPvHeads];  // (registers: the loops over it are unrolled to the kernel's most heads)
            const float* sr = sc + ((size_t)(m0 + min(row, nrows - 1)) * H + h_lo) * NK + (ok ? (j >= sp.j_lo ? sp.n_first + (j - sp.j_lo) : j) : 0);
#pragma unroll
            for (int g = 0; g < kPvHeads; ++g)
                p[g] = (ok && g < h_n) ? expf(sr[(size_t)g * NK] - s_M[row * H + h_lo + g]) * s_iZ[row * H + h_lo + g] : 0.0f;
            if (!talk) {  // no mixing matrix: every head keeps its own weights
#pragma unroll
                for (int g = 0; g < kPvHeads; ++g)
                    if (g < h_n) s_w[(g * 32 + row) * KP + kk] = p[g];
                continue;
            }
            for (int h = 0; h < H; ++h) {
                float wsum = 0.0f;
#pragma unroll
                for (int g = 0; g < kPvHeads; ++g) wsum = fmaf(g < H ? s_talk[h * H + g] : 0.0f, p[g], wsum);
                s_w[(h * 32 + row) * KP + kk] = wsum;
            }
        }
        __syncthreads();
        float vv[kPvUnits][kPvKeys / 2];  // the values of all the wave's units are requested before the first product
#pragma unroll
        for (int u = 0; u < kPvUnits; ++u) {
            const int unit = min(u0 + u, units - 1), h = unit / ctiles, c = (unit % ctiles) * 32 + r;
            const float* vcol = cache + (size_t)G * D + (size_t)(h / rep) * V + min(c, V - 1);
#pragma unroll
            for (int t = 0; t < kPvKeys / 2; ++t) vv[u][t] = c < V ? vcol[(size_t)s_row[kh * (kPvKeys / 2) + t] * cstride] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kPvUnits; ++u) {
            const int unit = u0 + u;
            if (unit < units) {
                const float* wrow = s_w + ((unit / ctiles - h_lo) * 32 + r) * KP + kh * (kPvKeys / 2);
#pragma unroll
                for (int t = 0; t < kPvKeys / 2; ++t) acc[u] = __builtin_amdgcn_mfma_f32_32x32x2f32(wrow[t], vv[u][t], acc[u], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < kPvUnits; ++u) {
        const int unit = u0 + u;
        if (unit < units) {
            const int h = unit / ctiles, c = (unit % ctiles) * 32 + r;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int qi = 8 * (i >> 2) + 4 * kh + (i & 3);
                if (qi < nrows && c < V) po[((size_t)(m0 + qi) * n_split + blockIdx.y) * H * V + (size_t)h * V + c] = acc[u][i];
            }
        }
    }
}

// gate != null: the heads' outputs are multiplied by sigmoid(gate[m][.]) * factor on their way out (a gated attention's last step)
__global__ __launch_bounds__(256) void window_merge_kernel(const float* po, int n_split, float* out, int ldo, int H, int V, const float* vfreq,
                                                           const int* row_pos, const float* gate, int ldg, float factor) {
    const int m = blockIdx.x;
    const float fpos = (float)row_pos[m];
    const float* base = po + (size_t)m * n_split * H * V;
    if (!vfreq) {  // unrotated values: the shares added in order, nothing to turn back
        for (int o = threadIdx.x; o < H * V; o += blockDim.x) {
            float a = 0.0f;
#pragma unroll 8
            for (int s2 = 0; s2 < n_split; ++s2) a += base[(size_t)s2 * H * V + o];
            if (gate) a *= sigmoid_f(gate[(size_t)m * ldg + o]) * factor;
            out[(size_t)m * ldo + o] = a;
        }
        return;
    }
    for (int p = threadIdx.x; p < H * V / 2; p += blockDim.x) {  // a pair of channels: (2i, 2i + 1) of a head
        float a = 0.0f, b = 0.0f;
#pragma unroll 8
        for (int s2 = 0; s2 < n_split; ++s2) {
            a += base[(size_t)s2 * H * V + 2 * p];
            b += base[(size_t)s2 * H * V + 2 * p + 1];
        }
        float sn, cs;
        sincosf(fpos * vfreq[p % (V / 2)], &sn, &cs);
        float oa = a * cs + b * sn, ob = b * cs - a * sn;
        if (gate) {
            oa *= sigmoid_f(gate[(size_t)m * ldg + 2 * p]) * factor;
            ob *= sigmoid_f(gate[(size_t)m * ldg + 2 * p + 1]) * factor;
        }
        out[(size_t)m * ldo + 2 * p] = oa;
        out[(size_t)m * ldo + 2 * p + 1] = ob;
    }
}

// ------------------------------------------------------------------------------------------------ gated linear recurrent unit
// Per entry and channel:  r = sigmoid(gr + br), i = sigmoid(gi + bi), a = exp(-8 r softplus(lam)),
// S = a S + sqrt(1 - a^2) i u,  out = S * gelu_tanh(y + by).  The recurrence is linear in S, so an entry's tokens are cut into
// kLruSegs stretches that run side by side: every stretch from a zero state (its end value and the product of its a), the
// start states down the stretches (one thread per channel), every stretch again from its true start, writing the outputs.
// A workgroup is 64 channels x kLruSegs stretches.  Entries of few tokens take one stretch, once.
constexpr int kLruSegs = 16;
__global__ __launch_bounds__(64 * kLruSegs) void rglru_scan_kernel(const float* u, int ldu, const float* gr, const float* gi, int ldg,
                                                                   const float* br, const float* bi, const float* lam, const float* y, int ldy,
                                                                   const float* by, float* out, int ldo, int C, float* state,
                                                                   size_t slot_stride, const int* ent_start, const int* ent_len,
                                                                   const int* ent_slot) {
    __shared__ float s_a[kLruSegs][64], s_b[kLruSegs][64];
    const int e = blockIdx.x, cl = threadIdx.x & 63, seg = threadIdx.x >> 6, c = blockIdx.y * 64 + cl;
    const int n = ent_len[e], m0 = ent_start[e];
    if (n <= 0) return;
    const bool ok = c < C;
    const int cc = ok ? c : 0;
    const bool cut = n >= 4 * kLruSegs;
    const int len = cut ? (n + kLruSegs - 1) / kLruSegs : n;
    const int t_lo = min(n, seg * len), t_hi = cut ? min(n, t_lo + len) : (seg == 0 ? n : 0);
    float* sp = state + (size_t)ent_slot[e] * slot_stride + cc;
    const float sl = softplus_f(lam[cc]), brc = br[cc], bic = bi[cc], byc = by[cc];
    auto coef = [&](int t, float& a, float& b) {
        const size_t m = (size_t)(m0 + t);
        a = expf(-8.0f * sigmoid_f(gr[m * ldg + cc] + brc) * sl);
        b = sqrtf(1.0f - a * a) * sigmoid_f(gi[m * ldg + cc] + bic) * u[m * ldu + cc];
    };
    float S = 0.0f;
    if (cut) {
        float A = 1.0f;
        for (int t = t_lo; t < t_hi; ++t) {
            float a, b;
            coef(t, a, b);
            S = fmaf(a, S, b);
            A *= a;
        }
        s_a[seg][cl] = A;
        s_b[seg][cl] = S;
        __syncthreads();
        if (seg == 0) {  // start state of every stretch, in place of its end value
            float run = *sp;
            for (int g2 = 0; g2 < kLruSegs; ++g2) {
                const float next = fmaf(s_a[g2][cl], run, s_b[g2][cl]);
                s_b[g2][cl] = run;
                run = next;
            }
            if (ok) *sp = run;
        }
        __syncthreads();
        S = s_b[seg][cl];
    } else {
        S = *sp;
    }
    for (int t = t_lo; t < t_hi; ++t) {
        float a, b;
        coef(t, a, b);
        S = fmaf(a, S, b);
        if (ok) out[(size_t)(m0 + t) * ldo + c] = S * gelu_tanh_f(y[(size_t)(m0 + t) * ldy + c] + byc);
    }
    if (!cut && seg == 0 && ok) *sp = S;
}

// y = (l / rms(l) * wl + r / rms(r) * wr) / 2, rows of W floats
__global__ __launch_bounds__(256) void pair_norm_mean_kernel(const float* l, const float* r, const float* wl, const float* wr, float eps, float* y,
                                                             int W) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const float *lr = l + (size_t)m * W, *rr = r + (size_t)m * W;
    float sa = 0.0f, sb = 0.0f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
        sa = fmaf(lr[i], lr[i], sa);
        sb = fmaf(rr[i], rr[i], sb);
    }
    sa = block_allsum(sa, s_red);
    sb = block_allsum(sb, s_red);
    const float ra = 1.0f / sqrtf(sa / (float)W + eps), rb = 1.0f / sqrtf(sb / (float)W + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) y[(size_t)m * W + i] = 0.5f * (lr[i] * ra * wl[i] + rr[i] * rb * wr[i]);
}

// ------------------------------------------------------------------------------------------------ gated delta rule
// In place on the rows of a step: q and k heads to unit length (q also times dim^-1/2), beta = sigmoid(.), and the decay
// g = exp(-exp(A_log[h]) * softplus(a + dt_bias)) per head and key channel.  One wave per vector / per stretch of elements.
__global__ __launch_bounds__(256) void delta_prep_kernel(float* qk, int ldqk, int G, int D, float* beta, int ldb, int H, float* dec, int ldd,
                                                         const float* a_log, const float* dt_bias) {
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int vsel = wave; vsel < 2 * G; vsel += 4) {  // q heads, then k heads
        float* p = qk + (size_t)m * ldqk + (size_t)vsel * D;
        float ss = 0.0f;
        for (int i = lane; i < D; i += 64) ss = fmaf(p[i], p[i], ss);
        ss = wave_allsum(ss);
        const float r = (1.0f / sqrtf(ss + 1e-6f)) * (vsel < G ? 1.0f / sqrtf((float)D) : 1.0f);
        for (int i = lane; i < D; i += 64) p[i] *= r;
    }
    for (int h = threadIdx.x; h < H; h += blockDim.x) beta[(size_t)m * ldb + h] = sigmoid_f(beta[(size_t)m * ldb + h]);
    for (int i = threadIdx.x; i < H * D; i += blockDim.x) {
        const float a = expf(a_log[i / D]);
        dec[(size_t)m * ldd + i] = expf(-a * softplus_f(dec[(size_t)m * ldd + i] + dt_bias[i]));
    }
}

// The recurrence of a head runs column by column of its state: u_c = beta (v_c - S[:, c] . k), S[:, c] += k u_c,
// o_c = S[:, c] . q touch no other column.  A column sits on the 16 lanes of one DPP row (lane i holds the RPL rows from i RPL
// on), a wave holds four columns, so the four column sums of a token are ONE row-wise reduction (four DPP adds); a workgroup's
// four waves take 16 neighbouring columns and the grid covers (entry, head, 16 columns).  The tokens' q, k, decay, values and
// beta reach the waves through the LDS, kDeltaBlock tokens at a time: the workgroup fetches a block together (few wide loads a
// thread) while it works on the block before — one barrier per block, none per token.
constexpr int kDeltaCols = 16;   // columns per workgroup
constexpr int kDeltaBlock = 8;   // tokens staged together
template <int RPL>
__global__ __launch_bounds__(256) void delta_scan_kernel(const float* qk, int ldqk, const float* v, int ldv, const float* beta, int ldb,
                                                         const float* dec, int ldd, float* out, int ldo, int H, int G, int D, int V,
                                                         float* state, size_t slot_stride, const int* ent_start, const int* ent_len,
                                                         const int* ent_slot) {
    extern __shared__ __attribute__((aligned(16))) float s_delta[];
    constexpr int Dp = 16 * RPL, TS = 3 * Dp + 20;  // a token's stage: q | k | g (Dp each) | v (16) | beta | pad
    constexpr int kDeltaFetch = (kDeltaBlock * TS + 255) / 256;  // loads a thread has in flight for a block
    const int e = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rl = lane & 15, cl = wave * 4 + (lane >> 4), c = blockIdx.z * kDeltaCols + cl;
    const int n = ent_len[e], m0 = ent_start[e];
    if (n <= 0) return;
    const bool col_ok = c < V;
    const int kvh = h / (H / G);
    float* Sg = state + (size_t)ent_slot[e] * slot_stride + (size_t)h * D * V;
    float S[RPL];
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int d = rl * RPL + r;
        S[r] = (d < D && col_ok) ? Sg[(size_t)d * V + c] : 0.0f;
    }
    // what a thread fetches for a block does not change from block to block: source, row stride and token are worked out once
    float pre[kDeltaFetch];
    const float* src[kDeltaFetch];
    int stride[kDeltaFetch], tok[kDeltaFetch];
#pragma unroll
    for (int i = 0; i < kDeltaFetch; ++i) {
        const int idx = tid + 256 * i, tt = idx / TS, o = idx % TS;
        src[i] = qk;
        stride[i] = 0;
        tok[i] = -1;
        if (tt < kDeltaBlock) {
            const int col = blockIdx.z * kDeltaCols + (o - 3 * Dp);
            if (o < Dp) {
                if (o < D) src[i] = qk + (size_t)kvh * D + o, stride[i] = ldqk, tok[i] = tt;
            } else if (o < 2 * Dp) {
                if (o - Dp < D) src[i] = qk + (size_t)(G + kvh) * D + (o - Dp), stride[i] = ldqk, tok[i] = tt;
            } else if (o < 3 * Dp) {
                if (o - 2 * Dp < D) src[i] = dec + (size_t)h * D + (o - 2 * Dp), stride[i] = ldd, tok[i] = tt;
            } else if (o < 3 * Dp + 16) {
                if (col < V) src[i] = v + (size_t)h * V + col, stride[i] = ldv, tok[i] = tt;
            } else if (o == 3 * Dp + 16) {
                src[i] = beta + h, stride[i] = ldb, tok[i] = tt;
            }
        }
    }
    auto fetch = [&](int t0) {
#pragma unroll
        for (int i = 0; i < kDeltaFetch; ++i)
            pre[i] = (tok[i] >= 0 && t0 + tok[i] < n) ? src[i][(size_t)(m0 + t0 + tok[i]) * stride[i]] : 0.0f;
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kDeltaFetch; ++i) {
            const int idx = tid + 256 * i;
            if (idx < kDeltaBlock * TS) s_delta[buf * kDeltaBlock * TS + idx] = pre[i];
        }
    };
    fetch(0);
    stash(0);
    for (int t0 = 0, blk = 0; t0 < n; t0 += kDeltaBlock, ++blk) {
        const bool more = t0 + kDeltaBlock < n;
        if (more) fetch(t0 + kDeltaBlock);
        __syncthreads();  // this block is staged; the other buffer has been consumed
        const float* sb = s_delta + (blk & 1) * kDeltaBlock * TS;
        const int nb = min(kDeltaBlock, n - t0);
#pragma unroll
        for (int i = 0; i < kDeltaBlock; ++i) {
            if (i >= nb) break;
            const float* st = sb + i * TS;
            float q[RPL], k[RPL], g[RPL];
            if constexpr (RPL % 4 == 0) {  // a lane's rows are consecutive: 16-byte LDS reads
#pragma unroll
                for (int r = 0; r < RPL; r += 4) {
                    const f32x4 a4 = *reinterpret_cast<const f32x4*>(st + rl * RPL + r);
                    const f32x4 b4 = *reinterpret_cast<const f32x4*>(st + Dp + rl * RPL + r);
                    const f32x4 c4 = *reinterpret_cast<const f32x4*>(st + 2 * Dp + rl * RPL + r);
                    q[r] = a4.x; q[r + 1] = a4.y; q[r + 2] = a4.z; q[r + 3] = a4.w;
                    k[r] = b4.x; k[r + 1] = b4.y; k[r + 2] = b4.z; k[r + 3] = b4.w;
                    g[r] = c4.x; g[r + 1] = c4.y; g[r + 2] = c4.z; g[r + 3] = c4.w;
                }
            } else {
#pragma unroll
                for (int r = 0; r < RPL; ++r) {
                    q[r] = st[rl * RPL + r];
                    k[r] = st[Dp + rl * RPL + r];
                    g[r] = st[2 * Dp + rl * RPL + r];
                }
            }
            const float vv = st[3 * Dp + cl], bt = st[3 * Dp + 16];
            float a = 0.0f;
#pragma unroll
            for (int r = 0; r < RPL; ++r) {
                S[r] *= g[r];
                a = fmaf(S[r], k[r], a);
            }
            const float u = bt * (vv - row16_allsum(a));
            a = 0.0f;
#pragma unroll
            for (int r = 0; r < RPL; ++r) {
                S[r] = fmaf(k[r], u, S[r]);
                a = fmaf(S[r], q[r], a);
            }
            a = row16_allsum(a);
            if (rl == 0 && col_ok) out[(size_t)(m0 + t0 + i) * ldo + (size_t)h * V + c] = a;
        }
        if (more) stash((blk + 1) & 1);
    }
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
        const int d = rl * RPL + r;
        if (d < D && col_ok) Sg[(size_t)d * V + c] = S[r];
    }
}

// one wave per (row, head) vector, in place: v / rms(v) * w * sigmoid(gate)
__global__ __launch_bounds__(256) void norm_gate_kernel(float* v, int ld, int rows_per_m, int width, int n_vec, const float* w, float eps,
                                                        const float* gate, int ldg, float factor, bool gate_silu) {
    const int vec = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (vec >= n_vec) return;
    const size_t m = vec / rows_per_m, hh = vec % rows_per_m;
    float* p = v + m * ld + hh * width;
    const float* gp = gate + m * ldg + hh * width;
    if (!w) {  // the gate and the factor only
        for (int i = lane; i < width; i += 64) p[i] = p[i] * sigmoid_f(gp[i]) * (gate_silu ? gp[i] : 1.0f) * factor;
        return;
    }
    float ss = 0.0f;
    for (int i = lane; i < width; i += 64) ss = fmaf(p[i], p[i], ss);
    ss = wave_allsum(ss);
    const float r = 1.0f / sqrtf(ss / (float)width + eps) * factor;
    for (int i = lane; i < width; i += 64) p[i] = p[i] * r * w[i] * sigmoid_f(gp[i]) * (gate_silu ? gp[i] : 1.0f);
}

// the same for wide vectors: a workgroup per vector
__global__ __launch_bounds__(256) void norm_gate_wide_kernel(float* v, int ld, int rows_per_m, int width, const float* w, float eps, const float* gate,
                                                             int ldg, float factor, bool gate_silu) {
    __shared__ float s_red[8];
    const size_t m = blockIdx.x / rows_per_m, hh = blockIdx.x % rows_per_m;
    float* p = v + m * ld + hh * width;
    const float* gp = gate + m * ldg + hh * width;
    float r = factor;
    if (w) {
        float ss = 0.0f;
        for (int i = threadIdx.x; i < width; i += blockDim.x) ss = fmaf(p[i], p[i], ss);
        ss = block_allsum(ss, s_red);
        r = 1.0f / sqrtf(ss / (float)width + eps) * factor;
    }
    for (int i = threadIdx.x; i < width; i += blockDim.x) p[i] = p[i] * r * (w ? w[i] : 1.0f) * sigmoid_f(gp[i]) * (gate_silu ? gp[i] : 1.0f);
}

// Decode steps (one row per entry) of the attention below: biases, the short convolutions of q | k | v with their tails moved
// on, both whole-projection norms, q written normed, keys and values into the cache — one launch.  A row's channels (up to
// 256 * kPrepRegs) and their tails (up to kPrepTaps - 1 inputs each) are requested up front and stay in registers; the two
// statistics share one pair of barriers.
constexpr int kPrepRegs = 8;
constexpr int kPrepTaps = 4;
__global__ __launch_bounds__(256) void conv_norm_prep_single_kernel(const float* __restrict__ in, int ld_in, float* __restrict__ qout, int ld_q, int HD,
                                                                    int GD, int GV, int taps, const float* __restrict__ cw,
                                                                    const float* __restrict__ pre_bias, float* __restrict__ tail, size_t slot_stride,
                                                                    const float* __restrict__ wq, const float* __restrict__ wk, float eps,
                                                                    const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                                    int page_tokens, float* __restrict__ cache) {
    __shared__ float s_red[2][4];
    const int m = blockIdx.x, CC = HD + GD + GV, K = taps - 1;
    const int pos = row_pos[m], slot = row_slot[m];
    const int page = page_table[(size_t)slot * max_pages + (pos / page_tokens) % max_pages];
    float* crow = cache + ((size_t)page * page_tokens + pos % page_tokens) * ((size_t)GD + GV);
    float* tl = tail + (size_t)slot * slot_stride;
    float cur[kPrepRegs], tv[kPrepRegs][kPrepTaps - 1], wv[kPrepRegs][kPrepTaps];
#pragma unroll
    for (int r = 0; r < kPrepRegs; ++r) {
        const int c = threadIdx.x + 256 * r;
        const bool ok = c < CC;
        cur[r] = ok ? in[(size_t)m * ld_in + c] + (pre_bias ? pre_bias[c] : 0.0f) : 0.0f;
#pragma unroll
        for (int j = 0; j < kPrepTaps - 1; ++j) tv[r][j] = (ok && j < K) ? tl[(size_t)j * CC + c] : 0.0f;
#pragma unroll
        for (int j = 0; j < kPrepTaps; ++j) wv[r][j] = (ok && j < taps) ? cw[(size_t)c * taps + j] : 0.0f;
    }
    float val[kPrepRegs];
    float sq = 0.0f, sk = 0.0f;
#pragma unroll
    for (int r = 0; r < kPrepRegs; ++r) {
        const int c = threadIdx.x + 256 * r;
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < kPrepTaps; ++j) {  // tap j < K reads the tail's input j (oldest first), tap K the current one
            float xin = cur[r];
#pragma unroll
            for (int u = 0; u < kPrepTaps - 1; ++u) xin = (j < K && u == j) ? tv[r][u] : xin;
            if (j <= K) acc = fmaf(wv[r][j], xin, acc);
        }
        val[r] = acc;
        if (c < HD) sq = fmaf(acc, acc, sq);
        else if (c < HD + GD) sk = fmaf(acc, acc, sk);
        if (c < CC) {
#pragma unroll
            for (int j = 0; j < kPrepTaps - 1; ++j)
                if (j < K) tl[(size_t)j * CC + c] = (j + 1 < K && j + 1 < kPrepTaps - 1) ? tv[r][(j + 1) % (kPrepTaps - 1)] : cur[r];
        }
    }
    sq = wave_allsum(sq);
    sk = wave_allsum(sk);
    if ((threadIdx.x & 63) == 0) {
        s_red[0][threadIdx.x >> 6] = sq;
        s_red[1][threadIdx.x >> 6] = sk;
    }
    __syncthreads();
    sq = (s_red[0][0] + s_red[0][1]) + (s_red[0][2] + s_red[0][3]);
    sk = (s_red[1][0] + s_red[1][1]) + (s_red[1][2] + s_red[1][3]);
    const float rq = 1.0f / sqrtf(sq / (float)HD + eps), rk = 1.0f / sqrtf(sk / (float)GD + eps);
#pragma unroll
    for (int r = 0; r < kPrepRegs; ++r) {
        const int c = threadIdx.x + 256 * r;
        if (c < HD) qout[(size_t)m * ld_q + c] = val[r] * rq * wq[c];
        else if (c < HD + GD) crow[c - HD] = val[r] * rk * wk[c - HD];
        else if (c < CC) crow[c - HD] = val[r];
    }
}

// Attention without rotation whose q and k are normed over the WHOLE projection (all heads together): one workgroup per row.
__global__ __launch_bounds__(256) void whole_norm_prep_kernel(float* qkv, int ld, int HD, int GD, int GV, const float* wq, const float* wk, float eps,
                                                              const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                              int page_tokens, float* cache) {
    __shared__ float s_red[8];
    const int m = blockIdx.x;
    const int pos = row_pos[m];
    const int page = page_table[(size_t)row_slot[m] * max_pages + (pos / page_tokens) % max_pages];
    float* crow = cache + ((size_t)page * page_tokens + pos % page_tokens) * ((size_t)GD + GV);
    float* q = qkv + (size_t)m * ld;
    const float *k = q + HD, *v = k + GD;
    float sq = 0.0f, sk = 0.0f;
    for (int i = threadIdx.x; i < HD; i += blockDim.x) sq = fmaf(q[i], q[i], sq);
    for (int i = threadIdx.x; i < GD; i += blockDim.x) sk = fmaf(k[i], k[i], sk);
    sq = block_allsum(sq, s_red);
    sk = block_allsum(sk, s_red);
    const float rq = 1.0f / sqrtf(sq / (float)HD + eps), rk = 1.0f / sqrtf(sk / (float)GD + eps);
    for (int i = threadIdx.x; i < HD; i += blockDim.x) q[i] = q[i] * rq * wq[i];
    for (int i = threadIdx.x; i < GD; i += blockDim.x) crow[i] = k[i] * rk * wk[i];
    for (int i = threadIdx.x; i < GV; i += blockDim.x) crow[GD + i] = v[i];
}

// Attention whose q and k are divided by their root mean square per head, and whose values reuse its un-normalised key projection: one
// workgroup per row, a wave per head (query heads, then key heads).  The query's factor grows with the logarithm of its position;
// the cache row receives the normed key heads and, behind them, the projected ones.
__global__ __launch_bounds__(256) void head_norm_prep_kernel(float* qk, int ld, int H, int G, int D, float eps, float qt_coef, int qt_every,
                                                             const int* row_pos, const int* row_slot, const int* page_table, int max_pages,
                                                             int page_tokens, float* cache) {
    const int m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pos = row_pos[m];
    const int page = page_table[(size_t)row_slot[m] * max_pages + (pos / page_tokens) % max_pages];
    float* crow = cache + ((size_t)page * page_tokens + pos % page_tokens) * ((size_t)2 * G * D);
    const float qf = qt_every > 0 ? 1.0f + qt_coef * logf((float)((pos + 1) / qt_every + 1)) : 1.0f;
    for (int u = wave; u < H + G; u += 4) {
        float* p = qk + (size_t)m * ld + (size_t)u * D;
        float ss = 0.0f;
        for (int i = lane; i < D; i += 64) ss = fmaf(p[i], p[i], ss);
        ss = wave_allsum(ss);
        const float r = 1.0f / sqrtf(ss / (float)D + eps);
        if (u < H) {
            for (int i = lane; i < D; i += 64) p[i] = p[i] * r * qf;
        } else {
            const int g = u - H;
            for (int i = lane; i < D; i += 64) {
                crow[(size_t)g * D + i] = p[i] * r;
                crow[(size_t)(G + g) * D + i] = p[i];
            }
        }
    }
}

}  // namespace

int launch_add_rows(float* x, const float* y, int M, int W, hipStream_t s) {
    const size_t n = (size_t)M * W;
    if (n == 0) return ZG_OK;
    add_rows_kernel<<<(unsigned)((n + 255) / 256), 256, 0, s>>>(x, y, n);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_causal_conv(const ConvArgs& a, int M, int n_entries, bool one_row_each, const int* row_off, const int* row_slot, const int* ent_start,
                       const int* ent_len, const int* ent_slot, hipStream_t s) {
    if (M <= 0 || a.C <= 0) return ZG_OK;
    ZG_REQUIRE(a.taps >= 1 && a.taps <= kMaxTaps, ZG_ERR_UNSUPPORTED, "convolution: %d taps (1 to %d)", a.taps, kMaxTaps);
    ZG_REQUIRE(a.in != a.out, ZG_ERR_ARG, "convolution: in place");
    const int bx = a.C >= 256 ? 256 : 64;
    causal_conv_kernel<<<dim3(M, (a.C + bx - 1) / bx), bx, 0, s>>>(a.in, a.ld_in, a.out, a.ld_out, a.C, a.taps, a.w, a.bias, a.pre_bias, a.flags, a.tail,
                                                                 a.slot_stride, row_off, row_slot, one_row_each ? 1 : 0);
    ZG_HIP(hipGetLastError());
    if (a.taps > 1 && !one_row_each) {
        conv_tail_kernel<<<dim3(n_entries, (a.C + bx - 1) / bx), bx, 0, s>>>(a.in, a.ld_in, a.C, a.taps, a.pre_bias, a.tail, a.slot_stride, ent_start,
                                                                           ent_len, ent_slot);
        ZG_HIP(hipGetLastError());
    }
    return ZG_OK;
}

int launch_norm_conv_single(float* x, const float* x0, const float* yl, const float* yr, const float* wl, const float* wr, const float* wb,
                            const float* wn, float eps, int M, int W, int taps, const float* cw, float* tail, size_t slot_stride,
                            const int* row_slot, float* out, hipStream_t s, bool* taken) {
    *taken = false;
    if (M <= 0 || W > 256 * kSingleRegs || taps < 1 || taps > kMaxTaps) return ZG_OK;
    norm_conv_single_kernel<<<M, 256, 0, s>>>(x, x0, yl, yr, wl, wr, wb, wn, eps, W, taps, cw, tail, slot_stride, row_slot, out);
    ZG_HIP(hipGetLastError());
    *taken = true;
    return ZG_OK;
}

int launch_window_prep(float* proj, int ld, int M, int H, int G, int D, int V, Rotary rot, const float* vfreq, const int* row_pos,
                       const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(V % 2 == 0 && rot.dims % 2 == 0 && rot.dims <= D, ZG_ERR_ARG, "windowed attention: %d value channels, %d of %d rotated", V, rot.dims, D);
    window_prep_kernel<<<M, 256, 0, s>>>(proj, ld, H, G, D, V, rot, vfreq, row_pos, row_slot, page_table, max_pages, page_tokens, cache);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_conv_norm_prep_single(const ConvArgs& a, float* qout, int ld_q, int M, int HD, int GD, int GV, const float* wq, const float* wk, float eps,
                                 const int* row_pos, const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache,
                                 hipStream_t s, bool* taken) {
    *taken = false;
    if (M <= 0 || HD + GD + GV > 256 * kPrepRegs || a.C != HD + GD + GV || a.taps < 1 || a.taps > kPrepTaps || a.bias || a.flags) return ZG_OK;
    conv_norm_prep_single_kernel<<<M, 256, 0, s>>>(a.in, a.ld_in, qout, ld_q, HD, GD, GV, a.taps, a.w, a.pre_bias, a.tail, a.slot_stride, wq, wk, eps,
                                                   row_pos, row_slot, page_table, max_pages, page_tokens, cache);
    ZG_HIP(hipGetLastError());
    *taken = true;
    return ZG_OK;
}

int launch_whole_norm_prep(float* qkv, int ld, int M, int HD, int GD, int GV, const float* wq, const float* wk, float eps, const int* row_pos,
                           const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    whole_norm_prep_kernel<<<M, 256, 0, s>>>(qkv, ld, HD, GD, GV, wq, wk, eps, row_pos, row_slot, page_table, max_pages, page_tokens, cache);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_window_attention(const float* q, int ldq, float* out, int ldo, int M, int H, int G, int D, int V, float scale, int window,
                            int keep_first, const float* sink, const float* talk, const float* vfreq, const int* row_pos, const int* row_slot,
                            const int* page_table, int max_pages, int page_tokens, const float* cache, hipStream_t s, ScoreShape shape) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(H >= 1 && H <= kWinMaxHeads && G >= 1 && H % G == 0, ZG_ERR_UNSUPPORTED, "windowed attention: %d heads on %d key heads (at most %d heads)",
               H, G, kWinMaxHeads);
    ZG_REQUIRE(H * V <= 256 * kWinAcc, ZG_ERR_UNSUPPORTED, "windowed attention: %d heads x %d value channels (at most %d together)", H, V,
               256 * kWinAcc);
    const size_t lds = ((size_t)H * D + 2 * (size_t)H * kWinTile + (size_t)H * H + (size_t)H * V) * sizeof(float);
    ZG_REQUIRE(lds <= 60 * 1024, ZG_ERR_UNSUPPORTED, "windowed attention: %d heads of %d + %d channels need %zu bytes of LDS", H, D, V, lds);
    window_attention_kernel<<<M, 256, lds, s>>>(q, ldq, out, ldo, H, G, D, V, scale, window, window > 0 ? keep_first : 0, sink, talk, vfreq, row_pos, row_slot, page_table,
                                                max_pages, page_tokens, cache, shape);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_head_norm_prep(float* qk, int ld, int M, int H, int G, int D, float eps, float qt_coef, int qt_every, const int* row_pos,
                          const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    ZG_REQUIRE(H >= 1 && G >= 1 && D >= 1 && ld >= (H + G) * D && qt_every >= 0, ZG_ERR_ARG, "attention prep: %d + %d heads of %d channels in rows of %d", H,
               G, D, ld);
    head_norm_prep_kernel<<<M, 256, 0, s>>>(qk, ld, H, G, D, eps, qt_coef, qt_every, row_pos, row_slot, page_table, max_pages, page_tokens, cache);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

size_t window_split_workspace(int rows, int H, int V, int key_capacity, int* n_split_out) {
    // shares of kMixTile keys: up to kWinSplits of them for steps of few rows (many workgroups per row), up to 16 for portions
    const int n_split = std::max(1, std::min(rows <= kGemvMaxRows ? kWinSplits : 16, (key_capacity + kMixTile - 1) / kMixTile));
    if (n_split_out) *n_split_out = n_split;
    return (size_t)rows * H * key_capacity + (size_t)rows * n_split * H * 2 + (size_t)rows * n_split * H * V;
}

int launch_window_attention_split(const float* q, int ldq, float* out, int ldo, int M, int H, int G, int D, int V, float scale, int window,
                                  int keep_first, const float* sink, const float* talk, const float* vfreq, const int* row_pos, const int* row_slot,
                                  const int* page_table, int max_pages, int page_tokens, const float* cache, int key_capacity, float* ws,
                                  size_t ws_floats, const int* ent_start, const int* ent_len, int n_entries, hipStream_t s, bool* taken,
                                  const float* out_gate, int ld_gate, float out_factor, ScoreShape shape) {
    *taken = false;
    if (M <= 0) return ZG_OK;
    const int keep = window > 0 ? keep_first : 0;
    if (const char* e = getenv("ZGPT2_LM_WINDOW_GENERAL"))  // test hook: every step through the general kernel
        if (atoi(e) != 0) return ZG_OK;
    int n_split = 1;
    const size_t need = window_split_workspace(M, H, V, key_capacity, &n_split);
    const int rpl = (D + 63) / 64;
    const size_t lds_a = ((size_t)H * 64 * rpl + (size_t)H * kScoreTile + 2 * (size_t)H) * sizeof(float);
    const size_t lds_b = (2 * (size_t)H * kMixTile + (size_t)H * H + 2 * (size_t)H) * sizeof(float);
    if (!ws || need > ws_floats || H > kWinMaxHeads || H % G != 0 || H * V > 256 * kWinAcc || D > 256 || (vfreq && V % 2 != 0) || lds_a > 60 * 1024 ||
        lds_b > 60 * 1024 || M > 65535)
        return ZG_OK;  // the general kernel takes it
    float* sc = ws;
    float* st = sc + (size_t)M * H * key_capacity;
    float* po = st + (size_t)M * n_split * H * 2;
    const dim3 grid(n_split, M);
    bool tiles = false;
    if (const char* e = getenv("ZGPT2_LM_WINDOW_TILES")) tiles = atoi(e) != 0;  // test hook: the tiled scores also for steps of few rows
    const bool tiled = (M > kGemvMaxRows || tiles) && D <= 128 && ent_start && getenv("ZGPT2_LM_WINDOW_NO_TILES") == nullptr;
    if (tiled) {
        // prompt portions: scores of 32 rows x 32 keys on the matrix cores, then the rows' statistics
        const int dh = (D + 1) / 2;
        const int max_tiles = (key_capacity + 31) / 32 + 2;
        const int ksplit = std::max(1, std::min(16, (max_tiles * G + 7) / 8));
        const dim3 tg((M + 31) / 32 + n_entries, ksplit);
#define ZG_WT(R)                                                                                                                                   \
    window_scores_mfma_kernel<R><<<tg, 256, 0, s>>>(q, ldq, H, G, D, V, scale, window, keep, ent_start, ent_len, n_entries, row_pos, row_slot, page_table, \
                                                    max_pages, page_tokens, cache, sc, key_capacity, shape)
        if (dh <= 8) ZG_WT(8);
        else if (dh <= 16) ZG_WT(16);
        else if (dh <= 32) ZG_WT(32);
        else ZG_WT(64);
#undef ZG_WT
        ZG_HIP(hipGetLastError());
        window_stats_kernel<<<M, 256, 0, s>>>(sc, key_capacity, H, window, keep, n_split, row_pos, st);
        ZG_HIP(hipGetLastError());
    } else {
#define ZG_WS(R)                                                                                                                              \
    window_scores_kernel<R><<<grid, 256, lds_a, s>>>(q, ldq, H, G, D, V, scale, window, keep, row_pos, row_slot, page_table, max_pages, page_tokens, cache, \
                                                     sc, key_capacity, st, shape)
    if (rpl <= 1) ZG_WS(1);
    else if (rpl <= 2) ZG_WS(2);
    else ZG_WS(4);
#undef ZG_WS
        ZG_HIP(hipGetLastError());
    }
    const bool mixes = talk != nullptr;  // (a mixing matrix: a workgroup weighs every head, else only those of its units)
    const int hs = mixes ? H : std::min(H, pv_block_heads((V + 31) / 32));
    const size_t lds_c = ((size_t)hs * 32 * (kPvKeys + 1) + (size_t)H * H + 64 * (size_t)H) * sizeof(float);
    if (tiled && (!mixes || H <= kPvHeads) && lds_c <= 60 * 1024) {  // the value product of 32 rows at a time on the matrix cores
        const int units = H * ((V + 31) / 32);
        const dim3 pg((M + 31) / 32 + n_entries, n_split, (units + 4 * kPvUnits - 1) / (4 * kPvUnits));
        window_mix_mfma_kernel<<<pg, 256, lds_c, s>>>(H, G, D, V, window, keep, sink, talk, ent_start, ent_len, n_entries, row_pos, row_slot, page_table,
                                                      max_pages, page_tokens, cache, sc, key_capacity, st, n_split, po);
    } else {
        window_mix_kernel<<<grid, 256, lds_b, s>>>(H, G, D, V, window, keep, sink, talk, row_pos, row_slot, page_table, max_pages, page_tokens, cache, sc,
                                                   key_capacity, st, po);
    }
    ZG_HIP(hipGetLastError());
    window_merge_kernel<<<M, 256, 0, s>>>(po, n_split, out, ldo, H, V, vfreq, row_pos, out_gate, ld_gate, out_factor);
    ZG_HIP(hipGetLastError());
    *taken = true;
    return ZG_OK;
}

int launch_rglru_scan(const float* u, int ldu, const float* gr, const float* gi, int ldg, const float* br, const float* bi, const float* lam,
                      const float* y, int ldy, const float* by, float* out, int ldo, int C, float* state, size_t slot_stride, const int* ent_start,
                      const int* ent_len, const int* ent_slot, int n_entries, hipStream_t s) {
    if (n_entries <= 0 || C <= 0) return ZG_OK;
    rglru_scan_kernel<<<dim3(n_entries, (C + 63) / 64), 64 * kLruSegs, 0, s>>>(u, ldu, gr, gi, ldg, br, bi, lam, y, ldy, by, out, ldo, C, state, slot_stride,
                                                                  ent_start, ent_len, ent_slot);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_pair_norm_mean(const float* l, const float* r, const float* wl, const float* wr, float eps, float* y, int M, int W, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    pair_norm_mean_kernel<<<M, 256, 0, s>>>(l, r, wl, wr, eps, y, W);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_delta_prep(float* qk, int ldqk, int G, int D, float* beta, int ldb, int H, float* dec, int ldd, const float* a_log,
                      const float* dt_bias, int M, hipStream_t s) {
    if (M <= 0) return ZG_OK;
    delta_prep_kernel<<<M, 256, 0, s>>>(qk, ldqk, G, D, beta, ldb, H, dec, ldd, a_log, dt_bias);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_delta_scan(const float* qk, int ldqk, const float* v, int ldv, const float* beta, int ldb, const float* dec, int ldd, float* out,
                      int ldo, int H, int G, int D, int V, float* state, size_t slot_stride, const int* ent_start, const int* ent_len,
                      const int* ent_slot, int n_entries, hipStream_t s) {
    if (n_entries <= 0) return ZG_OK;
    ZG_REQUIRE(D >= 1 && D <= 256 && V >= 1 && V <= 256 && G >= 1 && H % G == 0, ZG_ERR_UNSUPPORTED,
               "delta rule: %d heads on %d key heads, %d key and %d value channels per head (at most 256 each)", H, G, D, V);
    const int rpl = (D + 15) / 16;
    const int rp = rpl <= 1 ? 1 : rpl <= 2 ? 2 : rpl <= 4 ? 4 : rpl <= 8 ? 8 : 16;
    const size_t stage = (size_t)kDeltaBlock * (3 * 16 * rp + 20);
    const size_t lds = 2 * stage * sizeof(float);
    const dim3 grid(n_entries, H, (V + kDeltaCols - 1) / kDeltaCols);
#define ZG_DELTA(R) \
    delta_scan_kernel<R><<<grid, 256, lds, s>>>(qk, ldqk, v, ldv, beta, ldb, dec, ldd, out, ldo, H, G, D, V, state, slot_stride, ent_start, ent_len, ent_slot)
    if (rp == 1) ZG_DELTA(1);
    else if (rp == 2) ZG_DELTA(2);
    else if (rp == 4) ZG_DELTA(4);
    else if (rp == 8) ZG_DELTA(8);
    else ZG_DELTA(16);
#undef ZG_DELTA
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

int launch_norm_gate(float* v, int ld, int rows_per_m, int width, int M, const float* w, float eps, const float* gate, int ldg, hipStream_t s,
                     float factor, bool gate_silu) {
    const int n_vec = M * rows_per_m;
    if (n_vec <= 0) return ZG_OK;
    if (width > 256) {  // a workgroup per vector
        norm_gate_wide_kernel<<<n_vec, 256, 0, s>>>(v, ld, rows_per_m, width, w, eps, gate, ldg, factor, gate_silu);
        ZG_HIP(hipGetLastError());
        return ZG_OK;
    }
    norm_gate_kernel<<<(n_vec + 3) / 4, 256, 0, s>>>(v, ld, rows_per_m, width, n_vec, w, eps, gate, ldg, factor, gate_silu);
    ZG_HIP(hipGetLastError());
    return ZG_OK;
}

}  // namespace lm
}  // namespace zg
