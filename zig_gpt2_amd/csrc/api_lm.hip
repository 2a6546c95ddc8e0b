// api_lm.hip — the layered-model tier of the C ABI (include/zgpt2.h, zg_lm_*): decoder stacks described by data, served from
// state slots.  This file is the host side: the arena and the tensor table, the slot / page manager, the step function that
// turns a ragged batch of entries into portions of rows and launches the kernels of lm_linear.hip / lm_mix.hip / lm_moe.hip
// for every layer pass, and generation on top of the same step.
//
// Arena (one hipMalloc):
//   [ weights: bf16 matrices [out][in], fp32 vectors; fused where one product serves several projections:
//       hgrn2  qfv = q | f | v rows;   latent attention  dqkv = dq | dkv rows, uk kept TRANSPOSED per head ([H][kv_rank][dim]) so that
//       the query can be carried into the latent space by an ordinary [out][in] product;   experts  gu = gate | up rows per expert ]
//   [ state: token-shift rows [slot][pass][W] | recurrent states [slot][hgrn passes][H D V] | page table [slot][pages] |
//       latent cache per attention pass [page][token][kv_rank + rot_dim] ]          all fp32
//   [ scratch of one portion (max_step_tokens rows) | step metadata | logits ]
//
// Designs whose sublayers read h + conv(h) (canon_taps >= 1) and the mixers with convolutions or recurrences of their own keep, per
// slot and layer pass, one block of fp32 state: the tails of the input convolutions (the taps - 1 last inputs of both sublayers),
// the tail of the mixer's short convolutions, and its recurrent state (a vector per channel, or a matrix per head).  Windowed
// attention caches rotated keys and rotated values per token in the paged cache, through the same page table as the latents;
// pages that every attention pass's window has left behind return to the pool while the sequence is still open.
//
// Designs whose two sublayers stand side by side (x += mixer(norm1(x)) + ff(norm2(x))) leave a layer's sums open: the next
// layer's norm kernel adds them to x on its way (one statistic serves both norms), the last layer's are added in front of the
// final norm.  Their window + linear-attention mixer keeps, per slot and layer, the tail of the q / k / v convolutions and the
// [heads][dim][vdim] state of the linear attention in the same block of sequence state; its keys (normed) and values go to the
// paged cache as the other windowed attention's do.
//
// Designs whose norms are tanh(alpha v) * w + b keep a norm's three tensors together ([w | b | alpha]); such a norm needs no
// statistic, so the norm behind a sublayer, the residual sum (times the design's factor) and the norm in front of the next
// sublayer are one elementwise launch.  A layer that names another layer's weights is one more pass over that layer's tensors
// with separate cache and state.  Their gated linear attention keeps its [heads][dim][vdim] state in the block of sequence
// state; their attention caches the normed key heads and, as values, the projected ones.
//
// Latent attention runs in its absorbed form in prompts and in decoding alike: score_j = (W_uk^T q_nope) . c_j + q_rot . k_rot_j,
// out = W_uv (sum_j p_j c_j) — only the latent c_j and the rotated key part are cached, and a portion of a prompt needs nothing
// of the tokens before it but their cache rows.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <map>
#include <string>
#include <vector>

#include "lm_kernels.h"
#include "zg_kernels.h"

namespace zg {
namespace lm {

namespace {

enum { INIT_MATRIX = 0, INIT_OFFSET = 1, INIT_UNIT = 2, INIT_PLAIN = 3 };

struct Tensor {
    void* dev = nullptr;
    bool matrix = false;  // bf16 storage
    size_t rows = 0, cols = 0;
    size_t ld = 0;            // > 0: the rows lie ld elements apart (a column block of a wider matrix)
    int transpose_heads = 0;  // > 0: source [heads * d][cols] is stored as [heads][cols][d]
    int init = INIT_MATRIX;
    bool loaded = false;
};

struct LayerW {
    zg_lm_layer d;
    float *norm1 = nullptr, *norm1b = nullptr, *norm2 = nullptr, *norm2b = nullptr, *shift = nullptr;
    bf16_t *qfv = nullptr, *o = nullptr;
    float *fb = nullptr, *lower = nullptr, *hnorm = nullptr;
    bf16_t *dqkv = nullptr, *uq = nullptr, *ukT = nullptr, *uv = nullptr;
    float *dq_norm = nullptr, *dkv_norm = nullptr, *rot_freq = nullptr;
    float rot_amp = 1.0f;
    bf16_t *up = nullptr, *down = nullptr, *gu = nullptr, *edown = nullptr, *router = nullptr;
    float* correction = nullptr;  // the router's correction of the choice, or its bias (ZG_LM_ROUTE_TOP_LOGITS)
    // input convolutions of the two sublayers ([W][taps] fp32)
    float *canon1 = nullptr, *canon2 = nullptr;
    // parallel / delta rule: one fused projection (parallel: q | k | v | y | x;  delta rule: q | k | v | b | a1 | g1)
    bf16_t* wcat = nullptr;
    int n_cat = 0;
    // parallel
    bf16_t *ro = nullptr, *ra = nullptr, *ri = nullptr;
    float *sink = nullptr, *talk = nullptr, *left_out = nullptr, *right_out = nullptr, *yb = nullptr, *xb = nullptr, *convw = nullptr, *convb = nullptr;
    float *rab = nullptr, *rib = nullptr, *lam = nullptr, *vfreq = nullptr;
    // delta rule
    bf16_t *a2 = nullptr, *g2 = nullptr;
    float *a_log = nullptr, *dt_bias = nullptr;
    // window + linear pair: output projections of both branches side by side in one matrix ([W][H V + HR VR]), biases of q | k | v
    // in one vector, the whole-projection norms, the shared expert ([gate | up | gate logit] rows)
    bf16_t *ocat = nullptr, *sgu = nullptr, *sdown = nullptr;
    float *qkv_bias = nullptr, *qnorm = nullptr, *knorm = nullptr, *rnorm = nullptr, *obias = nullptr, *decay = nullptr;
    // gated linear attention: the bias of the decay's second step;  attention: the heads' slopes of the distance bias
    float *a2b = nullptr, *slopes = nullptr;
};

struct Pass {
    int layer = 0;
    size_t hgrn_off = 0;     // floats into a slot's recurrent-state block
    float* cache = nullptr;  // latent cache (or key / value cache) of this pass
    bool readd = false;      // the embedding output is added to x in front of this pass
    // floats into a slot's block of sequence state: tails of the two input convolutions, tail of the mixer's own convolution,
    // the mixer's recurrent state
    size_t canon1_off = 0, canon2_off = 0, conv_off = 0, rec_off = 0;
};

struct Slot {
    bool open = false;
    size_t len = 0;
    std::vector<int> pages;  // by position / page_tokens; -1: returned to the pool (behind every window)
    std::vector<int> ring;   // the device's view: page of position p at ring[(p / page_tokens) % max_pages]
    size_t first_live = 0;   // pages in front of this one have been returned
};

struct Bump {
    char* base;
    size_t off = 0;
    template <typename T>
    T* take(size_t n) {
        off = (off + 255) & ~(size_t)255;
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += n * sizeof(T);
        return p;
    }
};

struct Piece {  // the rows one entry contributes to one portion
    int slot;
    const int32_t* tok;
    int n;
    int pos0;
    std::vector<std::pair<int, size_t>> wants;  // (row inside the piece, output row)
};

struct Sampler {
    float temp;
    uint64_t seed;
    int32_t* tokens_out;  // host, indexed by output row
};

__global__ __launch_bounds__(256) void fill_kernel(void* dst, size_t n, uint64_t key, int kind, float std_, size_t cols, size_t ld) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint64_t z = key + (i + 1) * 0x9E3779B97F4A7C15ULL;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    z ^= z >> 31;
    const float s4 = (float)((int)((z & 0xFFFF) + ((z >> 16) & 0xFFFF) + ((z >> 32) & 0xFFFF) + (z >> 48)) - 131070) * (1.0f / 37837.227f);
    const float u = (float)(uint32_t)(z >> 40) * 5.9604644775390625e-08f;
    i = (i / cols) * ld + i % cols;
    if (kind == INIT_MATRIX) reinterpret_cast<bf16_t*>(dst)[i] = f32_to_bf16_rne(s4 * std_);
    else if (kind == INIT_OFFSET) reinterpret_cast<float*>(dst)[i] = s4 * 0.05f;
    else if (kind == INIT_UNIT) reinterpret_cast<float*>(dst)[i] = u;
    else reinterpret_cast<float*>(dst)[i] = 1.0f + s4 * 0.05f;
}

__global__ __launch_bounds__(256) void zero_kernel(float* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.0f;
}

__global__ __launch_bounds__(256) void ones_kernel(float* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 1.0f;
}

}  // namespace
}  // namespace lm
}  // namespace zg

using namespace zg;
using namespace zg::lm;

struct zg_lm {
    zg_lm_config cfg;
    std::vector<LayerW> layers;
    std::vector<Pass> passes;
    std::map<std::string, Tensor> tensors;
    int device = 0;
    hipStream_t stream = nullptr;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    char* arena = nullptr;
    size_t arena_bytes = 0;
    bool f32 = false;
    int W = 0, V = 0, MS = 0, NS = 0, P = 0, max_pages = 0, n_pages = 0, logit_rows = 0, n_passes = 0;
    // weights outside the layers
    bf16_t *embed = nullptr, *head = nullptr;
    float* final_norm = nullptr;
    // state
    float* shift_state = nullptr;  // [NS][passes][W]
    float* hgrn_state = nullptr;   // [NS][hgrn_floats]
    size_t hgrn_floats = 0;
    float* seq_state = nullptr;  // [NS][seq_floats]: convolution tails and recurrent states of the passes that have them
    size_t seq_floats = 0;
    int canon = 0;        // taps of the sublayers' input convolution (0: token shift)
    int keep_tokens = 0;  // > 0: no attention pass looks further back than this many tokens ...
    int keep_first = 0;   // ... except at the first keep_first tokens of the sequence, which some pass keeps in sight
    int keep_pages = 0;   // pages that hold those first tokens: never returned while the sequence is open
    float embed_scale = 1.0f;
    bool side = false;          // ZG_LM_SIDE_BY_SIDE
    bool tanh_norms = false;    // ZG_LM_TANH_NORMS: every norm pointer is a block [w | b | alpha]
    float res_mult = 1.0f;      // ... and a sublayer's normed output enters the residual sum times this
    float* embed_norm = nullptr;  // ZG_LM_EMBED_NORM
    float* pos_freq = nullptr;  // ZG_LM_SINUSOID_POSITIONS: frequency of every pair of channels
    int* page_table = nullptr;  // [NS][max_pages]
    std::vector<Slot> slots;
    std::vector<int> free_pages;
    // scratch
    float *x = nullptr, *h = nullptr, *y = nullptr, *proj = nullptr, *cq = nullptr, *q = nullptr, *qa = nullptr, *ctx = nullptr, *o = nullptr, *u = nullptr;
    float *gu_buf = nullptr, *hb = nullptr, *ye = nullptr, *wt = nullptr, *last_h = nullptr, *hn = nullptr, *logits = nullptr;
    float *row_max = nullptr, *samp_ws = nullptr, *samp_u = nullptr, *amax_val = nullptr;
    int* amax_idx = nullptr;
    float *attn_ws = nullptr, *scan_ws = nullptr, *win_ws = nullptr;
    size_t win_ws_floats = 0;
    float *x0 = nullptr, *hc = nullptr, *y2 = nullptr, *ta = nullptr, *tb = nullptr, *tc = nullptr, *td = nullptr;
    size_t scan_ws_floats = 0;
    size_t attn_ws_floats = 0;
    int *pick = nullptr, *grp_off = nullptr, *sorted = nullptr, *inv = nullptr, *tok_out = nullptr, *flag = nullptr;
    int* meta = nullptr;    // device: ids | pos | slot | prev | last-entry | want rows | entry start | entry len | entry slot
    int* h_meta = nullptr;  // pinned twin
    float* h_logits = nullptr;  // pinned [logit_rows][V]
    int* h_small = nullptr;     // pinned: sampled tokens [logit_rows], fault flag
    float* h_u = nullptr;       // pinned uniforms [logit_rows]
    float* trace = nullptr;
    size_t trace_floats = 0;
    float last_step_ms = 0.0f, last_decode_ms = 0.0f;
    bool use_graph = true;
    int step_keys = 0;  // positions the longest sequence of the running portion has reached (what its rows can see at most)
    // by rows of the step (one per entry) and, where whole-context attention splits a row's keys into shares, by the length bucket
    // of the longest sequence (512, 1024, ... tokens): a share then holds a few dozen keys at any length
    static constexpr int kKeyBuckets = 24;
    hipGraphExec_t decode_graph[kGemvMaxRows + 1][kKeyBuckets] = {};
    bool whole_context = false;  // some pass attends over the whole sequence through the split kernels
    int bucket_keys = 0;         // key capacity of the running decode step's bucket
};

namespace {

// ids | pos | slot | prev | last-entry | want rows | entry start | entry len | entry slot | place of the row inside its entry
size_t meta_ints(const zg_lm* g) { return (size_t)7 * g->MS + (size_t)3 * g->NS; }
size_t meta_row_off(const zg_lm* g) { return (size_t)6 * g->MS + (size_t)3 * g->NS; }

// Everything that lives in the arena, in one place: called once with a null base to measure and once to place.
void layout(zg_lm* g, Bump& b) {
    const size_t W = g->W, V = g->V, MS = g->MS, NS = g->NS;
    auto& T = g->tensors;
    T.clear();
    auto mat = [&](const std::string& name, bf16_t* base, size_t row0, size_t rows, size_t cols, int transpose_heads = 0) {
        Tensor t;
        t.dev = base ? base + row0 * cols : nullptr;
        t.matrix = true;
        t.rows = rows;
        t.cols = cols;
        t.transpose_heads = transpose_heads;
        t.init = INIT_MATRIX;
        T[name] = t;
    };
    // columns [col0, col0 + cols) of a matrix whose rows are ld wide
    auto mat_cols = [&](const std::string& name, bf16_t* base, size_t rows, size_t ld, size_t col0, size_t cols) {
        Tensor t;
        t.dev = base ? base + col0 : nullptr;
        t.matrix = true;
        t.rows = rows;
        t.cols = cols;
        t.ld = ld;
        t.init = INIT_MATRIX;
        T[name] = t;
    };
    auto vec = [&](const std::string& name, float*& p, size_t n, int init) {
        p = b.take<float>(n);
        Tensor t;
        t.dev = p;
        t.rows = 1;
        t.cols = n;
        t.init = init;
        T[name] = t;
    };
    auto vec_at = [&](const std::string& name, float* base, size_t off, size_t n, int init) {
        Tensor t;
        t.dev = base ? base + off : nullptr;
        t.rows = 1;
        t.cols = n;
        t.init = init;
        T[name] = t;
    };
    // a norm tanh(alpha v) * w + b: its three tensors side by side
    auto norm3 = [&](const std::string& name, float*& p) {
        p = b.take<float>(2 * W + 1);
        vec_at(name, p, 0, W, INIT_PLAIN);
        vec_at(name + ".b", p, W, W, INIT_OFFSET);
        vec_at(name + ".alpha", p, 2 * W, 1, INIT_PLAIN);
    };
    const bool tn = g->tanh_norms;
    const size_t taps = g->canon;
    g->embed = b.take<bf16_t>(V * W);
    mat("embed", g->embed, 0, V, W);
    if (tn && (g->cfg.flags & ZG_LM_EMBED_NORM)) norm3("embed.norm", g->embed_norm);
    if (g->cfg.flags & ZG_LM_TIED_HEAD) {
        g->head = g->embed;
    } else {
        g->head = b.take<bf16_t>(V * W);
        mat("head", g->head, 0, V, W);
    }
    if (tn) norm3("final.norm", g->final_norm);
    else vec("final.norm", g->final_norm, W, g->side ? INIT_PLAIN : INIT_OFFSET);
    if (g->cfg.flags & ZG_LM_SINUSOID_POSITIONS) g->pos_freq = b.take<float>((W + 1) / 2);
    size_t max_t = 1, max_win = 0, max_win_few = 0;
    size_t max_proj = 1, max_qr = 1, max_q = 1, max_qa = 1, max_ctx = 1, max_o = 1, max_ff = 1, max_assign = 1, max_gu = 1, max_hb = 1, max_e = 1, max_att_part = 0, max_scan = 0;
    for (size_t i = 0; i < g->layers.size(); ++i) {
        LayerW& L = g->layers[i];
        const zg_lm_layer& d = L.d;
        const std::string p = "l" + std::to_string(i) + ".";
        if (d.weights_of > 0) continue;  // another layer's tensors
        if (tn) {
            norm3(p + "norm1", L.norm1);
            norm3(p + "norm1b", L.norm1b);
        } else vec(p + "norm1", L.norm1, W, g->side ? INIT_PLAIN : INIT_OFFSET);
        if (g->side || tn) {
        } else {
            vec(p + "norm1b", L.norm1b, W, INIT_OFFSET);
            if (taps == 0) vec(p + "shift", L.shift, W, INIT_UNIT);
            else vec(p + "canon1", L.canon1, W * taps, INIT_OFFSET);
        }
        const size_t H = d.heads, D = d.dim, Vd = d.vdim;
        if (d.mixer == ZG_LM_MIX_PARALLEL) {
            const size_t G = d.kv_heads, C = d.lru_width, NB = d.lru_blocks, BS = C / NB, HV = H * Vd;
            const size_t NP = H * D + G * D + G * Vd + 2 * C;
            L.n_cat = (int)NP;
            L.wcat = b.take<bf16_t>(NP * W);
            mat(p + "mix.left.q", L.wcat, 0, H * D, W);
            mat(p + "mix.left.k", L.wcat, H * D, G * D, W);
            mat(p + "mix.left.v", L.wcat, H * D + G * D, G * Vd, W);
            mat(p + "mix.right.y", L.wcat, H * D + G * D + G * Vd, C, W);
            mat(p + "mix.right.x", L.wcat, H * D + G * D + G * Vd + C, C, W);
            vec(p + "mix.left.sink", L.sink, H, INIT_OFFSET);
            vec(p + "mix.left.talk", L.talk, H * H, INIT_UNIT);
            L.o = b.take<bf16_t>(W * HV);
            mat(p + "mix.left.o", L.o, 0, W, HV);
            vec(p + "mix.left.out", L.left_out, W, INIT_PLAIN);
            vec(p + "mix.right.out", L.right_out, W, INIT_PLAIN);
            vec(p + "mix.right.y.b", L.yb, C, INIT_OFFSET);
            vec(p + "mix.right.x.b", L.xb, C, INIT_OFFSET);
            vec(p + "mix.right.conv", L.convw, C * d.lru_conv, INIT_OFFSET);
            vec(p + "mix.right.conv.b", L.convb, C, INIT_OFFSET);
            L.ra = b.take<bf16_t>(NB * BS * BS);
            mat(p + "mix.right.ra", L.ra, 0, NB * BS, BS);
            L.ri = b.take<bf16_t>(NB * BS * BS);
            mat(p + "mix.right.ri", L.ri, 0, NB * BS, BS);
            vec(p + "mix.right.ra.b", L.rab, C, INIT_OFFSET);
            vec(p + "mix.right.ri.b", L.rib, C, INIT_OFFSET);
            vec(p + "mix.right.lam", L.lam, C, INIT_OFFSET);
            L.ro = b.take<bf16_t>(W * C);
            mat(p + "mix.right.o", L.ro, 0, W, C);
            L.rot_freq = b.take<float>(std::max<size_t>(1, d.rot_dims / 2));
            L.vfreq = b.take<float>(std::max<size_t>(1, Vd / 2));
            max_proj = std::max(max_proj, NP);
            max_o = std::max(max_o, HV);
            max_t = std::max(max_t, C);
            const int cap = d.window > 0 ? d.window : g->max_pages * g->P;
            max_win = std::max(max_win, window_split_workspace((int)MS, (int)H, (int)Vd, cap, nullptr));
            max_win_few = std::max(max_win_few, window_split_workspace(kGemvMaxRows, (int)H, (int)Vd, cap, nullptr));
        } else if (d.mixer == ZG_LM_MIX_WINDOW_LINEAR) {
            const size_t G = d.kv_heads, HD = H * D, GD = G * D, GV = G * Vd, CC = HD + GD + GV, HV = H * Vd;
            const size_t HR = d.lin_heads, HRD = HR * d.lin_dim, HRV = HR * d.lin_vdim, NP = CC + HV + 2 * HRD + 2 * HRV;
            const size_t ct = std::max(1, d.conv);
            L.n_cat = (int)NP;
            L.wcat = b.take<bf16_t>(NP * W);  // left q | k | v | gate, right q | k | v | gate
            const std::string l = p + "mix.left.", r = p + "mix.right.";
            mat(l + "q", L.wcat, 0, HD, W);
            mat(l + "k", L.wcat, HD, GD, W);
            mat(l + "v", L.wcat, HD + GD, GV, W);
            mat(l + "g", L.wcat, CC, HV, W);
            mat(r + "q", L.wcat, CC + HV, HRD, W);
            mat(r + "k", L.wcat, CC + HV + HRD, HRD, W);
            mat(r + "v", L.wcat, CC + HV + 2 * HRD, HRV, W);
            mat(r + "g", L.wcat, CC + HV + 2 * HRD + HRV, HRV, W);
            L.qkv_bias = b.take<float>(CC);
            vec_at(l + "q.b", L.qkv_bias, 0, HD, INIT_OFFSET);
            vec_at(l + "k.b", L.qkv_bias, HD, GD, INIT_OFFSET);
            vec_at(l + "v.b", L.qkv_bias, HD + GD, GV, INIT_OFFSET);
            L.convw = b.take<float>(CC * ct);  // without a convolution: one tap of weight one, set at creation
            if (d.conv >= 1) {
                vec_at(l + "q.conv", L.convw, 0, HD * ct, INIT_OFFSET);
                vec_at(l + "k.conv", L.convw, HD * ct, GD * ct, INIT_OFFSET);
                vec_at(l + "v.conv", L.convw, (HD + GD) * ct, GV * ct, INIT_OFFSET);
            }
            vec(l + "q.norm", L.qnorm, HD, INIT_PLAIN);
            vec(l + "k.norm", L.knorm, GD, INIT_PLAIN);
            L.ocat = b.take<bf16_t>(W * (HV + HRV));
            mat_cols(l + "o", L.ocat, W, HV + HRV, 0, HV);
            mat_cols(r + "o", L.ocat, W, HV + HRV, HV, HRV);
            vec(l + "o.b", L.obias, W, INIT_OFFSET);
            vec(r + "norm", L.rnorm, HRV, INIT_PLAIN);
            vec(r + "decay", L.decay, HR, INIT_UNIT);
            max_proj = std::max(max_proj, NP);
            max_o = std::max(max_o, HV + HRV);
            max_t = std::max(max_t, std::max(CC, W));
            max_scan = std::max(max_scan, HRD * d.lin_vdim + HRD);
            const int cap = d.window > 0 ? d.window + d.keep_first : g->max_pages * g->P;
            max_win = std::max(max_win, window_split_workspace((int)MS, (int)H, (int)Vd, cap, nullptr));
            max_win_few = std::max(max_win_few, window_split_workspace(kGemvMaxRows, (int)H, (int)Vd, cap, nullptr));
        } else if (d.mixer == ZG_LM_MIX_CHANNEL_DELTA) {
            const size_t G = d.kv_heads, HV = H * Vd, CC = 2 * G * D + HV, RA = d.decay_rank, RG = d.gate_rank;
            const size_t NP = CC + H + RA + RG;
            L.n_cat = (int)NP;
            L.wcat = b.take<bf16_t>(NP * W);
            mat(p + "mix.q", L.wcat, 0, G * D, W);
            mat(p + "mix.k", L.wcat, G * D, G * D, W);
            mat(p + "mix.v", L.wcat, 2 * G * D, HV, W);
            mat(p + "mix.b", L.wcat, CC, H, W);
            mat(p + "mix.a1", L.wcat, CC + H, RA, W);
            mat(p + "mix.g1", L.wcat, CC + H + RA, RG, W);
            L.convw = b.take<float>(CC * d.conv);
            vec_at(p + "mix.q.conv", L.convw, 0, G * D * d.conv, INIT_OFFSET);
            vec_at(p + "mix.k.conv", L.convw, G * D * d.conv, G * D * d.conv, INIT_OFFSET);
            vec_at(p + "mix.v.conv", L.convw, 2 * G * D * d.conv, HV * d.conv, INIT_OFFSET);
            L.a2 = b.take<bf16_t>(H * D * RA);
            mat(p + "mix.a2", L.a2, 0, H * D, RA);
            L.g2 = b.take<bf16_t>(HV * RG);
            mat(p + "mix.g2", L.g2, 0, HV, RG);
            vec(p + "mix.A_log", L.a_log, H, INIT_OFFSET);
            vec(p + "mix.dt_bias", L.dt_bias, H * D, INIT_OFFSET);
            vec(p + "mix.norm", L.hnorm, Vd, INIT_PLAIN);
            L.o = b.take<bf16_t>(W * HV);
            mat(p + "mix.o", L.o, 0, W, HV);
            max_proj = std::max(max_proj, NP);
            max_t = std::max(max_t, std::max(CC, std::max(H * D, HV)));
        } else if (d.mixer == ZG_LM_MIX_GLA) {
            const size_t HD = H * D, HV = H * Vd, RA = d.decay_rank, NP = 2 * HD + 2 * HV + RA;
            L.n_cat = (int)NP;
            L.wcat = b.take<bf16_t>(NP * W);  // q | k | v | gate | the decay's first step
            mat(p + "mix.q", L.wcat, 0, HD, W);
            mat(p + "mix.k", L.wcat, HD, HD, W);
            mat(p + "mix.v", L.wcat, 2 * HD, HV, W);
            mat(p + "mix.g", L.wcat, 2 * HD + HV, HV, W);
            mat(p + "mix.a1", L.wcat, 2 * HD + 2 * HV, RA, W);
            L.a2 = b.take<bf16_t>(HD * RA);
            mat(p + "mix.a2", L.a2, 0, HD, RA);
            vec(p + "mix.a2.b", L.a2b, HD, INIT_OFFSET);
            vec(p + "mix.norm", L.hnorm, Vd, INIT_PLAIN);
            L.o = b.take<bf16_t>(W * HV);
            mat(p + "mix.o", L.o, 0, W, HV);
            max_proj = std::max(max_proj, NP);
            max_t = std::max(max_t, HD);
            max_scan = std::max(max_scan, HD * Vd + HD);
            max_o = std::max(max_o, HV);
        } else if (d.mixer == ZG_LM_MIX_ATTENTION) {
            const size_t G = d.kv_heads, HD = H * D, GD = G * D, NP = HD + GD;
            L.n_cat = (int)NP;
            L.wcat = b.take<bf16_t>(NP * W);  // q | k (values reuse the key projection)
            mat(p + "mix.q", L.wcat, 0, HD, W);
            mat(p + "mix.k", L.wcat, HD, GD, W);
            L.o = b.take<bf16_t>(W * HD);
            mat(p + "mix.o", L.o, 0, W, HD);
            L.slopes = b.take<float>(H);
            max_proj = std::max(max_proj, NP);
            max_o = std::max(max_o, HD);
            // (a portion's score rows are as long as its longest sequence: what exceeds the bound below takes the general kernel)
            const int cap = g->max_pages * g->P;
            max_win = std::max(max_win, std::min(window_split_workspace((int)MS, (int)H, (int)D, cap, nullptr), (size_t)1 << 29));
            max_win_few = std::max(max_win_few, window_split_workspace(kGemvMaxRows, (int)H, (int)D, cap, nullptr));
        } else if (d.mixer == ZG_LM_MIX_HGRN2) {
            const size_t HD = H * D, HV = H * Vd;
            L.qfv = b.take<bf16_t>((2 * HD + HV) * W);
            mat(p + "mix.q", L.qfv, 0, HD, W);
            mat(p + "mix.f", L.qfv, HD, HD, W);
            mat(p + "mix.v", L.qfv, 2 * HD, HV, W);
            vec(p + "mix.f.b", L.fb, HD, INIT_OFFSET);
            vec(p + "mix.lower", L.lower, HD, INIT_UNIT);
            vec(p + "mix.norm", L.hnorm, Vd, INIT_PLAIN);
            L.o = b.take<bf16_t>(W * HV);
            mat(p + "mix.o", L.o, 0, W, HV);
            max_proj = std::max(max_proj, 2 * HD + HV);
            max_scan = std::max(max_scan, H * D * Vd + H * D);
            max_o = std::max(max_o, HV);
        } else {
            const size_t R = d.rot_dim, KR = d.kv_rank, QR = d.q_rank, HV = H * Vd;
            L.dqkv = b.take<bf16_t>((QR + KR + R) * W);
            mat(p + "mix.dq", L.dqkv, 0, QR, W);
            mat(p + "mix.dkv", L.dqkv, QR, KR + R, W);
            vec(p + "mix.dq.norm", L.dq_norm, QR, INIT_PLAIN);
            vec(p + "mix.dkv.norm", L.dkv_norm, KR, INIT_PLAIN);
            L.uq = b.take<bf16_t>(H * (D + R) * QR);
            mat(p + "mix.uq", L.uq, 0, H * (D + R), QR);
            L.ukT = b.take<bf16_t>(H * KR * D);
            mat(p + "mix.uk", L.ukT, 0, H * D, KR, (int)H);
            L.uv = b.take<bf16_t>(HV * KR);
            mat(p + "mix.uv", L.uv, 0, HV, KR);
            L.o = b.take<bf16_t>(W * HV);
            mat(p + "mix.o", L.o, 0, W, HV);
            L.rot_freq = b.take<float>(std::max<size_t>(1, d.rot_dims / 2));
            max_proj = std::max(max_proj, QR + KR + R);
            max_qr = std::max(max_qr, QR);
            max_q = std::max(max_q, H * (D + R));
            max_qa = std::max(max_qa, H * (KR + R));
            max_ctx = std::max(max_ctx, H * KR);
            max_att_part = std::max(max_att_part, H * (KR + 2));
            max_o = std::max(max_o, HV);
        }
        if (d.ff != ZG_LM_FF_NONE && tn) {
            norm3(p + "norm2", L.norm2);
            norm3(p + "norm2b", L.norm2b);
        } else if (d.ff != ZG_LM_FF_NONE) {
            vec(p + "norm2", L.norm2, W, g->side ? INIT_PLAIN : INIT_OFFSET);
            if (!g->side) vec(p + "norm2b", L.norm2b, W, INIT_OFFSET);
            if (taps && !g->side) vec(p + "canon2", L.canon2, W * taps, INIT_OFFSET);
        }
        const size_t F = d.ff_width;
        if (d.ff == ZG_LM_FF_DENSE) {
            L.up = b.take<bf16_t>(F * W);
            mat(p + "mlp.up", L.up, 0, F, W);
            L.down = b.take<bf16_t>(W * F);
            mat(p + "mlp.down", L.down, 0, W, F);
            max_ff = std::max(max_ff, F);
        } else if (d.ff == ZG_LM_FF_MOE) {
            const size_t E = d.experts, UF = d.ff_act == ZG_LM_ACT_GELU ? F : 2 * F;  // rows of an expert's first matrix
            L.gu = b.take<bf16_t>(E * UF * W);
            L.edown = b.take<bf16_t>(E * W * F);
            for (size_t e = 0; e < E; ++e) {
                const std::string q = p + "mlp.e" + std::to_string(e) + ".";
                if (UF == 2 * F) mat(q + "gate", L.gu, e * 2 * F, F, W);
                mat(q + "up", L.gu, e * UF + (UF - F), F, W);
                mat(q + "down", L.edown, e * W, W, F);
            }
            L.router = b.take<bf16_t>(E * W);
            mat(p + "mlp.router", L.router, 0, E, W);
            if (d.router != ZG_LM_ROUTE_SIGMOID_INPUT)
                vec(p + (d.router == ZG_LM_ROUTE_TOP_LOGITS ? "mlp.router.b" : "mlp.correction"), L.correction, E, INIT_OFFSET);
            if (d.shared_width > 0) {  // the shared expert: gate | up rows and, behind them, the row of its gate logit (clipped form)
                const size_t S = d.shared_width;
                L.sgu = b.take<bf16_t>((2 * S + 1) * W);
                mat(p + "mlp.shared.gate", L.sgu, 0, S, W);
                mat(p + "mlp.shared.up", L.sgu, S, S, W);
                if (d.ff_act == ZG_LM_ACT_GLU_CLIPPED) mat(p + "mlp.shared.sg", L.sgu, 2 * S, 1, W);
                L.sdown = b.take<bf16_t>(W * S);
                mat(p + "mlp.shared.down", L.sdown, 0, W, S);
                max_t = std::max(max_t, std::max(2 * S + 1, W));
            }
            max_assign = std::max(max_assign, (size_t)d.top);
            max_gu = std::max(max_gu, (size_t)d.top * UF);
            max_hb = std::max(max_hb, (size_t)d.top * F);
            max_e = std::max(max_e, E);
        }
    }
    // state
    g->shift_state = b.take<float>(NS * g->n_passes * W);
    size_t hg = 0;
    for (Pass& ps : g->passes) {
        const zg_lm_layer& d = g->layers[ps.layer].d;
        if (d.mixer == ZG_LM_MIX_HGRN2) {
            ps.hgrn_off = hg;
            hg += (size_t)d.heads * d.dim * d.vdim;
        }
    }
    g->hgrn_floats = hg;
    g->hgrn_state = b.take<float>(std::max<size_t>(1, NS * hg));
    size_t sq = 0;
    for (Pass& ps : g->passes) {
        const zg_lm_layer& d = g->layers[ps.layer].d;
        if (taps > 1) {
            ps.canon1_off = sq;
            sq += (taps - 1) * W;
            if (d.ff != ZG_LM_FF_NONE) {
                ps.canon2_off = sq;
                sq += (taps - 1) * W;
            }
        }
        if (d.mixer == ZG_LM_MIX_PARALLEL) {
            ps.conv_off = sq;
            sq += (size_t)(d.lru_conv - 1) * d.lru_width;
            ps.rec_off = sq;
            sq += d.lru_width;
        } else if (d.mixer == ZG_LM_MIX_CHANNEL_DELTA) {
            ps.conv_off = sq;
            sq += (size_t)(d.conv - 1) * (2 * d.kv_heads * d.dim + d.heads * d.vdim);
            ps.rec_off = sq;
            sq += (size_t)d.heads * d.dim * d.vdim;
        } else if (d.mixer == ZG_LM_MIX_WINDOW_LINEAR) {
            ps.conv_off = sq;
            sq += (size_t)(std::max(1, d.conv) - 1) * ((size_t)d.heads * d.dim + (size_t)d.kv_heads * (d.dim + d.vdim));
            ps.rec_off = sq;
            sq += (size_t)d.lin_heads * d.lin_dim * d.lin_vdim;
        } else if (d.mixer == ZG_LM_MIX_GLA) {
            ps.rec_off = sq;
            sq += (size_t)d.heads * d.dim * d.vdim;
        }
    }
    g->seq_floats = sq;
    g->seq_state = b.take<float>(std::max<size_t>(1, NS * sq));
    g->page_table = b.take<int>(NS * g->max_pages);
    for (Pass& ps : g->passes) {
        const zg_lm_layer& d = g->layers[ps.layer].d;
        if (d.mixer == ZG_LM_MIX_LATENT_ATTENTION) ps.cache = b.take<float>((size_t)g->n_pages * g->P * (d.kv_rank + d.rot_dim));
        if (d.mixer == ZG_LM_MIX_PARALLEL || d.mixer == ZG_LM_MIX_WINDOW_LINEAR)
            ps.cache = b.take<float>((size_t)g->n_pages * g->P * d.kv_heads * (d.dim + d.vdim));
        if (d.mixer == ZG_LM_MIX_ATTENTION) ps.cache = b.take<float>((size_t)g->n_pages * g->P * d.kv_heads * 2 * d.dim);
    }
    // scratch
    g->x = b.take<float>(MS * W);
    g->h = b.take<float>(MS * W);
    g->y = b.take<float>(MS * W);
    g->x0 = b.take<float>(MS * W);
    g->hc = b.take<float>(MS * W);
    g->y2 = b.take<float>(MS * W);
    g->ta = b.take<float>(MS * max_t);
    g->tb = b.take<float>(MS * max_t);
    g->tc = b.take<float>(MS * max_t);
    g->td = b.take<float>(MS * max_t);
    g->proj = b.take<float>(MS * max_proj);
    g->cq = b.take<float>(MS * max_qr);
    g->q = b.take<float>(MS * max_q);
    g->qa = b.take<float>(MS * max_qa);
    g->ctx = b.take<float>(MS * max_ctx);
    g->o = b.take<float>(MS * max_o);
    g->u = b.take<float>(MS * max_ff);
    g->gu_buf = b.take<float>(MS * max_gu);
    g->hb = b.take<float>(MS * max_hb);
    g->ye = b.take<float>(MS * max_assign * W);
    g->wt = b.take<float>(MS * max_assign);
    g->pick = b.take<int>(MS * max_assign);
    g->sorted = b.take<int>(MS * max_assign);
    g->inv = b.take<int>(MS * max_assign);
    g->grp_off = b.take<int>(max_e + 1);
    g->scan_ws_floats = (MS / 32 + 1 + NS) * max_scan;  // a state per chunk of the chunked recurrences (chunks of 64 or 32 tokens)
    g->scan_ws = b.take<float>(std::max<size_t>(1, g->scan_ws_floats));
    g->attn_ws_floats = (size_t)kGemvMaxRows * kAttnSplits * max_att_part;
    g->attn_ws = b.take<float>(std::max<size_t>(1, g->attn_ws_floats));
    // scores and partial sums of the split windowed attention: up to 2 GiB for a whole portion, else for steps of few rows only
    // (longer steps of such a model then take the general kernel)
    if (max_win > ((size_t)1 << 29)) max_win = 0;
    max_win = std::max(max_win, max_win_few);
    if (max_win > ((size_t)1 << 29)) max_win = 0;
    g->win_ws_floats = max_win;
    g->win_ws = b.take<float>(std::max<size_t>(1, max_win));
    g->last_h = b.take<float>((size_t)g->n_passes * NS * W);
    g->hn = b.take<float>((size_t)g->logit_rows * W);
    g->logits = b.take<float>((size_t)g->logit_rows * V);
    g->row_max = b.take<float>(g->logit_rows);
    g->samp_ws = b.take<float>(sample_workspace_floats(g->logit_rows));
    g->samp_u = b.take<float>(g->logit_rows);
    g->tok_out = b.take<int>(g->logit_rows);
    g->amax_val = b.take<float>((size_t)g->logit_rows * kArgmaxParts);
    g->amax_idx = b.take<int>((size_t)g->logit_rows * kArgmaxParts);
    g->flag = b.take<int>(16);
    g->meta = b.take<int>(meta_ints(g));
}

// YaRN blend of the rotary frequencies (host, double): pairs below `lo` keep their frequency, pairs above `hi` are slowed by
// `factor`, a linear ramp between; the amplitude factor multiplies cos and sin.
void rotary_table(const zg_lm_layer& d, std::vector<float>& freq, float& amp) {
    const int dims = d.rot_dims, half = dims / 2;
    freq.resize(std::max(1, half));
    amp = 1.0f;
    if (d.rot_scaled == ZG_LM_ROT_BANDS) {  // by wavelength: short waves stay, long waves are slowed, a linear blend between
        for (int i = 0; i < half; ++i) {
            const double f = pow((double)d.rot_base, -2.0 * i / dims), wave = 2.0 * M_PI / f;
            const double orig = d.rot_original, high = d.rot_fast, low = d.rot_slow;
            double out = f;
            if (wave < orig / high) out = f;
            else if (wave > orig / low) out = f / d.rot_factor;
            else {
                const double t = (orig / wave - low) / (high - low);
                out = (1.0 - t) * f / d.rot_factor + t * f;
            }
            freq[i] = (float)out;
        }
        return;
    }
    double lo = 0, hi = 0;
    if (d.rot_scaled) {
        auto corr = [&](double t) { return dims * log((double)d.rot_original / (2.0 * M_PI * t)) / (2.0 * log((double)d.rot_base)); };
        lo = std::max(floor(corr(d.rot_fast)), 0.0);
        hi = std::min(ceil(corr(d.rot_slow)), (double)dims - 1.0);
        amp = (float)(0.1 * log((double)d.rot_factor) + 1.0);
    }
    for (int i = 0; i < half; ++i) {
        double f = pow((double)d.rot_base, -2.0 * i / dims);
        if (d.rot_scaled) {
            const double ramp = std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001)));
            f = f / d.rot_factor * ramp + f * (1.0 - ramp);
        }
        freq[i] = (float)f;
    }
}

int check_layer(const zg_lm_layer& d, size_t i, unsigned flags) {
    ZG_REQUIRE(d.mixer >= ZG_LM_MIX_HGRN2 && d.mixer <= ZG_LM_MIX_ATTENTION, ZG_ERR_ARG, "layer %zu: unknown mixer %d", i, d.mixer);
    ZG_REQUIRE(d.heads >= 1 && d.dim >= 1 && d.vdim >= 1, ZG_ERR_ARG, "layer %zu: heads %d dim %d vdim %d", i, d.heads, d.dim, d.vdim);
    if (d.mixer == ZG_LM_MIX_PARALLEL || d.mixer == ZG_LM_MIX_CHANNEL_DELTA || d.mixer == ZG_LM_MIX_WINDOW_LINEAR || d.mixer == ZG_LM_MIX_ATTENTION)
        ZG_REQUIRE(d.kv_heads >= 1 && d.heads % d.kv_heads == 0, ZG_ERR_ARG, "layer %zu: %d heads on %d key heads", i, d.heads, d.kv_heads);
    if (d.mixer == ZG_LM_MIX_PARALLEL) {
        ZG_REQUIRE(d.vdim % 2 == 0, ZG_ERR_ARG, "layer %zu: %d value channels per head cannot be rotated in pairs", i, d.vdim);
        ZG_REQUIRE(d.rot_dims >= 0 && d.rot_dims % 2 == 0 && d.rot_dims <= d.dim, ZG_ERR_ARG, "layer %zu: %d rotated dimensions of %d", i, d.rot_dims,
                   d.dim);
        ZG_REQUIRE(d.rot_base > 0.0f && d.window >= 0, ZG_ERR_ARG, "layer %zu: rotary base %f, window %d", i, d.rot_base, d.window);
        ZG_REQUIRE(!d.rot_scaled || (d.rot_factor > 0.0f && d.rot_original > 0.0f && d.rot_fast > 0.0f && d.rot_slow > 0.0f &&
                                     (d.rot_scaled != ZG_LM_ROT_BANDS || d.rot_fast != d.rot_slow)),
                   ZG_ERR_ARG, "layer %zu: rotary scaling constants", i);
        ZG_REQUIRE(d.lru_width >= 1 && d.lru_blocks >= 1 && d.lru_width % d.lru_blocks == 0 && d.lru_conv >= 1 && d.lru_conv <= 16, ZG_ERR_ARG,
                   "layer %zu: recurrent unit of %d channels in %d blocks, %d taps", i, d.lru_width, d.lru_blocks, d.lru_conv);
    } else if (d.mixer == ZG_LM_MIX_WINDOW_LINEAR) {
        ZG_REQUIRE(flags & ZG_LM_SIDE_BY_SIDE, ZG_ERR_UNSUPPORTED, "layer %zu: the window + linear pair is built for side-by-side sublayers", i);
        ZG_REQUIRE(d.window >= 0 && d.keep_first >= 0 && d.conv >= 0 && d.conv <= 16, ZG_ERR_ARG, "layer %zu: window %d, %d first tokens kept, %d taps", i,
                   d.window, d.keep_first, d.conv);
        ZG_REQUIRE(d.lin_heads >= 1 && d.lin_dim >= 1 && d.lin_vdim >= 1 && d.lin_dim <= 256, ZG_ERR_UNSUPPORTED,
                   "layer %zu: linear attention of %d heads, %d key and %d value channels (at most 256 key channels)", i, d.lin_heads, d.lin_dim,
                   d.lin_vdim);
    } else if (d.mixer == ZG_LM_MIX_CHANNEL_DELTA) {
        ZG_REQUIRE(d.conv >= 1 && d.conv <= 16 && d.decay_rank >= 1 && d.gate_rank >= 1, ZG_ERR_ARG, "layer %zu: %d taps, inner sizes %d and %d", i,
                   d.conv, d.decay_rank, d.gate_rank);
        ZG_REQUIRE(d.dim <= 256 && d.vdim <= 256, ZG_ERR_UNSUPPORTED, "layer %zu: a delta-rule state of %d x %d per head (at most 256 each)", i, d.dim,
                   d.vdim);
    } else if (d.mixer == ZG_LM_MIX_HGRN2) {
        ZG_REQUIRE(d.dim <= 256, ZG_ERR_UNSUPPORTED, "layer %zu: %d key channels per head of the recurrence (at most 256)", i, d.dim);
    } else if (d.mixer == ZG_LM_MIX_GLA) {
        ZG_REQUIRE(d.dim <= 256, ZG_ERR_UNSUPPORTED, "layer %zu: %d key channels per head of the recurrence (at most 256)", i, d.dim);
        ZG_REQUIRE(d.tau > 0.0f && d.decay_rank >= 1, ZG_ERR_ARG, "layer %zu: decay root %g, inner size %d of its projection", i, d.tau, d.decay_rank);
    } else if (d.mixer == ZG_LM_MIX_ATTENTION) {
        ZG_REQUIRE(d.vdim == d.dim, ZG_ERR_ARG, "layer %zu: values reuse the key projection, so %d value channels cannot differ from %d key channels", i, d.vdim,
                   d.dim);
        ZG_REQUIRE(d.softcap >= 0.0f && d.qtemp_every >= 0 && d.window == 0, ZG_ERR_ARG, "layer %zu: score cap %g, query factor every %d, window %d", i,
                   d.softcap, d.qtemp_every, d.window);
    } else {
        ZG_REQUIRE(d.rot_dim >= 0 && d.kv_rank >= 1 && d.q_rank >= 1, ZG_ERR_ARG, "layer %zu: rot_dim %d kv_rank %d q_rank %d", i, d.rot_dim,
                   d.kv_rank, d.q_rank);
        ZG_REQUIRE(d.rot_dims >= 0 && d.rot_dims % 2 == 0 && d.rot_dims <= d.rot_dim, ZG_ERR_ARG, "layer %zu: %d rotated dimensions of %d", i,
                   d.rot_dims, d.rot_dim);
        ZG_REQUIRE(d.kv_rank + d.rot_dim <= 1024, ZG_ERR_UNSUPPORTED, "layer %zu: %d cached dimensions per token (at most 1024)", i,
                   d.kv_rank + d.rot_dim);
        ZG_REQUIRE(d.rot_dims == 0 || d.rot_base > 0.0f, ZG_ERR_ARG, "layer %zu: rotary base %f", i, d.rot_base);
        ZG_REQUIRE(!d.rot_scaled || (d.rot_factor > 0.0f && d.rot_original > 0.0f && d.rot_fast > 0.0f && d.rot_slow > 0.0f), ZG_ERR_ARG,
                   "layer %zu: rotary scaling constants must be positive", i);
    }
    ZG_REQUIRE(d.ff == ZG_LM_FF_NONE || d.ff == ZG_LM_FF_DENSE || d.ff == ZG_LM_FF_MOE, ZG_ERR_ARG, "layer %zu: unknown feed-forward %d", i, d.ff);
    ZG_REQUIRE(d.ff == ZG_LM_FF_NONE || d.ff_width >= 1, ZG_ERR_ARG, "layer %zu: feed-forward width %d", i, d.ff_width);
    ZG_REQUIRE(d.ff != ZG_LM_FF_MOE || (d.experts >= 1 && d.experts <= 256 && d.top >= 1 && d.top <= d.experts), ZG_ERR_UNSUPPORTED,
               "layer %zu: %d experts, %d chosen (at most 256 experts)", i, d.experts, d.top);
    ZG_REQUIRE(d.ff_act >= ZG_LM_ACT_GLU_SILU && d.ff_act <= ZG_LM_ACT_GLU_CLIPPED && d.router >= ZG_LM_ROUTE_SOFTMAX_ALL &&
                   d.router <= ZG_LM_ROUTE_SIGMOID_GROUPS,
               ZG_ERR_ARG, "layer %zu: expert activation %d, router rule %d", i, d.ff_act, d.router);
    if (d.ff == ZG_LM_FF_MOE && !(flags & ZG_LM_SIDE_BY_SIDE))
        ZG_REQUIRE(d.ff_act != ZG_LM_ACT_GLU_CLIPPED && d.router != ZG_LM_ROUTE_SIGMOID_INPUT && (d.shared_width == 0 || (flags & ZG_LM_TANH_NORMS)),
                   ZG_ERR_UNSUPPORTED,
                   "layer %zu: the clipped activation and the input-weighted router are built for side-by-side sublayers, a shared expert for those or "
                   "for the norms without statistics",
                   i);
    if (d.ff == ZG_LM_FF_MOE && d.router == ZG_LM_ROUTE_SIGMOID_GROUPS) {
        const int ng = std::max(1, d.route_groups), nk = d.route_keep >= 1 ? d.route_keep : ng;
        ZG_REQUIRE(d.experts % ng == 0 && nk <= ng && d.top <= nk * (d.experts / ng) && d.route_scale >= 0.0f, ZG_ERR_ARG,
                   "layer %zu: %d experts in %d groups, %d groups kept, %d chosen, weight factor %g", i, d.experts, ng, nk, d.top, d.route_scale);
    }
    if (d.ff == ZG_LM_FF_MOE && d.ff_act == ZG_LM_ACT_GLU_CLIPPED)
        ZG_REQUIRE(d.ff_limit > 0.0f && (d.shared_width == 0 || d.shared_limit > 0.0f), ZG_ERR_ARG, "layer %zu: clip %g (shared expert: %g)", i, d.ff_limit,
                   d.shared_limit);
    ZG_REQUIRE(d.shared_width >= 0 && (d.shared_width == 0 || d.ff_act == ZG_LM_ACT_GLU_CLIPPED ||
                                       (d.ff_act == ZG_LM_ACT_GLU_SILU && (flags & ZG_LM_TANH_NORMS))),
               ZG_ERR_UNSUPPORTED, "layer %zu: a shared expert needs a gated activation", i);
    return ZG_OK;
}

// The kernels of one portion, from the embedding to the commit of the token-shift rows: launches only, every per-step value
// (tokens, positions, slots, page tables) is read from device memory — so for a given number of rows and entries the sequence
// is the same every step and can be replayed from a captured graph (decode steps: one row per entry).
int enqueue_layers(zg_lm* g, int M, int n_ent, bool capturing, bool single) {
    hipStream_t s = g->stream;
    const int W = g->W, MS = g->MS, NS = g->NS;
    const int *d_ids = g->meta, *d_pos = d_ids + MS, *d_slot = d_pos + MS, *d_prev = d_slot + MS, *d_last = d_prev + MS, *d_want = d_last + MS;
    const int *d_estart = d_want + MS, *d_elen = d_estart + NS, *d_eslot = d_elen + NS;
    const int* d_off = g->meta + meta_row_off(g);
    const bool f32 = g->f32;
    const float eps = g->cfg.norm_eps;
    const bool few = M <= kGemvMaxRows;
    const bool canon = g->canon >= 1;
    const bool readd = (g->cfg.flags & ZG_LM_LOOP_READD) && g->cfg.loop_times > 1;
    ZG_TRY(launch_embed(g->embed, d_ids, g->x, readd ? g->x0 : nullptr, g->embed_scale, M, W, g->V, g->flag, d_pos, g->pos_freq, s));
    const bool side = g->side;
    const bool tnorm = g->tanh_norms;
    // side-by-side sublayers: the sums a layer leaves for the next layer's norm kernel to add
    OpenSums pend;
    auto copy_trace = [&](int p) -> int {
        if (g->trace && !capturing && (size_t)(p + 1) * M * W <= g->trace_floats) {
            ZG_HIP(hipMemcpyAsync(g->trace + (size_t)p * M * W, g->x, (size_t)M * W * sizeof(float), hipMemcpyDeviceToHost, s));
            ZG_HIP(hipStreamSynchronize(s));
        }
        return ZG_OK;
    };
    // h + conv(h) of a sublayer's input, and the tail of the slots moved on
    auto input_conv = [&](const float* w, size_t off) -> int {
        ConvArgs c;
        c.in = g->h; c.ld_in = W; c.out = g->hc; c.ld_out = W; c.C = W; c.taps = g->canon; c.w = w; c.flags = CONV_RESIDUAL;
        c.tail = g->seq_state + off; c.slot_stride = g->seq_floats;
        return launch_causal_conv(c, M, n_ent, single, d_off, d_slot, d_estart, d_elen, d_eslot, s);
    };
    bool h_ready = false;  // g->h already holds this pass's shifted norm (written by the previous pass's fused tail)
    if (tnorm) {  // the norm behind the embedding (in place) and the first pass's norm; every later one rides behind a sublayer's sum
        ZG_TRY(launch_tanh_norm(g->x, g->embed_norm, g->layers[g->passes[0].layer].norm1, nullptr, g->h, M, W, s));
        h_ready = true;
    }
    for (int p = 0; p < g->n_passes; ++p) {
        const Pass& ps = g->passes[p];
        const LayerW& L = g->layers[ps.layer];
        const zg_lm_layer& d = L.d;
        const int H = d.heads, D = d.dim, Vd = d.vdim;
        bool hc_ready = false;  // one launch has done everything up to the mixer's input (decode steps)
        if (side) {  // what the layer before left open, and both norms of this layer from one statistic
            ZG_TRY(launch_norm_two(g->x, pend, L.norm1, d.ff != ZG_LM_FF_NONE ? L.norm2 : nullptr, eps, g->h, g->hc, M, W, s));
            pend = OpenSums();
            h_ready = true;
        }
        if (canon && single && !h_ready)
            ZG_TRY(launch_norm_conv_single(g->x, ps.readd ? g->x0 : nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, L.norm1, eps, M, W, g->canon,
                                           L.canon1, g->seq_state + ps.canon1_off, g->seq_floats, d_slot, g->hc, s, &hc_ready));
        if (ps.readd && !hc_ready) ZG_TRY(launch_add_rows(g->x, g->x0, M, W, s));
        if (!h_ready && !hc_ready)
            ZG_TRY(launch_norm_shift(g->x, L.norm1, canon ? nullptr : L.shift, eps, g->h, M, W, d_prev, d_slot, g->shift_state + (size_t)p * W,
                                     (size_t)g->n_passes * W, canon ? nullptr : d_last, g->last_h + (size_t)p * NS * W, s));
        h_ready = false;
        const float* hin = g->h;  // what the sublayer reads
        if (canon) {
            if (!hc_ready) ZG_TRY(input_conv(L.canon1, ps.canon1_off));
            hin = g->hc;
        }
        // one row per entry: the pass's last sum is fused with the next pass's norm + shift (tail below)
        auto tail = [&](const float* y, const float* yexp, const float* weight, int top, const float* wb) -> int {
            if (!single || p + 1 >= g->n_passes || canon) return ZG_OK;
            const LayerW& N = g->layers[g->passes[p + 1].layer];
            return launch_sum_norm_shift(g->x, y, yexp, weight, top, wb, N.norm1, N.shift, eps, g->h, M, W, d_slot, g->shift_state + (size_t)(p + 1) * W,
                                         (size_t)g->n_passes * W, d_last, g->last_h + (size_t)(p + 1) * NS * W, s, &h_ready);
        };
        Linear lin;
        bool mid_done = false;  // x, and the feed-forward's input in g->hc, are already there
        if (d.mixer == ZG_LM_MIX_WINDOW_LINEAR) {
            const int G = d.kv_heads, HD = H * D, GD = G * D, GV = G * Vd, CC = HD + GD + GV, HV = H * Vd;
            const int HR = d.lin_heads, DR = d.lin_dim, VR = d.lin_vdim, HRD = HR * DR, HRV = HR * VR, NP = L.n_cat, OC = HV + HRV;
            const int og = CC, orq = CC + HV, org = orq + 2 * HRD + HRV;  // columns of the left gate, the right q | k | v, the right gate
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.wcat; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            // left: biases and convolutions of q | k | v at once, the whole-projection norms, keys and values into the cache
            ConvArgs cv;
            cv.in = g->proj; cv.ld_in = NP; cv.out = g->ta; cv.ld_out = CC; cv.C = CC; cv.taps = std::max(1, d.conv); cv.w = L.convw;
            cv.pre_bias = L.qkv_bias; cv.tail = g->seq_state + ps.conv_off; cv.slot_stride = g->seq_floats;
            bool prepped = false;  // decode steps: convolution, norms and cache rows in one launch
            if (single)
                ZG_TRY(launch_conv_norm_prep_single(cv, g->ta, CC, M, HD, GD, GV, L.qnorm, L.knorm, eps, d_pos, d_slot, g->page_table, g->max_pages, g->P,
                                                    ps.cache, s, &prepped));
            if (!prepped) {
                ZG_TRY(launch_causal_conv(cv, M, n_ent, single, d_off, d_slot, d_estart, d_elen, d_eslot, s));
                ZG_TRY(launch_whole_norm_prep(g->ta, CC, M, HD, GD, GV, L.qnorm, L.knorm, eps, d_pos, d_slot, g->page_table, g->max_pages, g->P, ps.cache,
                                              s));
            }
            bool split = false;
            ZG_TRY(launch_window_attention_split(g->ta, CC, g->o, OC, M, H, G, D, Vd, d.scale, d.window, d.keep_first, nullptr, nullptr, nullptr, d_pos,
                                                 d_slot, g->page_table, g->max_pages, g->P, ps.cache,
                                                 d.window > 0 ? d.window + d.keep_first : g->max_pages * g->P, g->win_ws, g->win_ws_floats, d_estart,
                                                 d_elen, n_ent, s, &split, g->proj + og, NP, d.left_scale));  // (the gate where the shares meet)
            if (!split) {
                ZG_TRY(launch_window_attention(g->ta, CC, g->o, OC, M, H, G, D, Vd, d.scale, d.window, d.keep_first, nullptr, nullptr, nullptr, d_pos,
                                               d_slot, g->page_table, g->max_pages, g->P, ps.cache, s));
                ZG_TRY(launch_norm_gate(g->o, OC, 1, HV, M, nullptr, eps, g->proj + og, NP, s, d.left_scale));
            }
            // right: the recurrence on silu(q | k | v), the heads normed together and gated
            ZG_TRY(launch_hgrn2_scan(g->proj + orq, NP, g->o + HV, OC, g->seq_state + ps.rec_off, g->seq_floats, d_estart, d_elen, d_eslot, n_ent, M, HR,
                                     DR, VR, nullptr, nullptr, g->scan_ws, g->scan_ws_floats, s, L.decay));
            ZG_TRY(launch_norm_gate(g->o + HV, OC, 1, HRV, M, L.rnorm, eps, g->proj + org, NP, s, d.right_scale));
            lin = Linear();  // both output projections at once: [c_l left | c_r right] against [left.o | right.o]
            lin.A = g->o; lin.lda = OC; lin.B = L.ocat; lin.ldb = OC; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = OC;
            ZG_TRY(launch_linear(lin, f32, s));
        } else if (d.mixer == ZG_LM_MIX_PARALLEL) {
            const int G = d.kv_heads, C = d.lru_width, NB = d.lru_blocks, BS = C / NB, HV = H * Vd, NP = L.n_cat;
            const int oy = H * D + G * D + G * Vd, ox = oy + C;  // columns of the two branches of the recurrent unit
            const Rotary rot{L.rot_freq, d.rot_dims, 1.0f};
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.wcat; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            // left: attention inside the window
            ZG_TRY(launch_window_prep(g->proj, NP, M, H, G, D, Vd, rot, L.vfreq, d_pos, d_slot, g->page_table, g->max_pages, g->P, ps.cache, s));
            bool split = false;
            ZG_TRY(launch_window_attention_split(g->proj, NP, g->o, HV, M, H, G, D, Vd, d.scale, d.window, 0, L.sink, L.talk, L.vfreq, d_pos, d_slot,
                                                 g->page_table, g->max_pages, g->P, ps.cache, d.window > 0 ? d.window : g->max_pages * g->P, g->win_ws,
                                                 g->win_ws_floats, d_estart, d_elen, n_ent, s, &split));
            if (!split)
                ZG_TRY(launch_window_attention(g->proj, NP, g->o, HV, M, H, G, D, Vd, d.scale, d.window, 0, L.sink, L.talk, L.vfreq, d_pos, d_slot,
                                               g->page_table, g->max_pages, g->P, ps.cache, s));
            lin = Linear();
            lin.A = g->o; lin.lda = HV; lin.B = L.o; lin.ldb = HV; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HV;
            ZG_TRY(launch_linear(lin, f32, s));
            // right: convolution, gates block by block, the recurrence
            ConvArgs cv;
            cv.in = g->proj + ox; cv.ld_in = NP; cv.out = g->ta; cv.ld_out = C; cv.C = C; cv.taps = d.lru_conv; cv.w = L.convw; cv.bias = L.convb;
            cv.pre_bias = L.xb; cv.tail = g->seq_state + ps.conv_off; cv.slot_stride = g->seq_floats;
            ZG_TRY(launch_causal_conv(cv, M, n_ent, single, d_off, d_slot, d_estart, d_elen, d_eslot, s));
            for (int which = 0; which < 2; ++which) {
                lin = Linear();
                lin.A = g->ta; lin.lda = C; lin.a_zoff = BS; lin.B = which ? L.ri : L.ra; lin.ldb = BS; lin.b_zoff = (long long)BS * BS;
                lin.C = which ? g->tc : g->tb; lin.ldc = C; lin.c_zoff = BS; lin.M = M; lin.N = BS; lin.K = BS; lin.nz = NB;
                ZG_TRY(launch_linear(lin, f32, s));
            }
            ZG_TRY(launch_rglru_scan(g->ta, C, g->tb, g->tc, C, L.rab, L.rib, L.lam, g->proj + oy, NP, L.yb, g->td, C, C, g->seq_state + ps.rec_off,
                                     g->seq_floats, d_estart, d_elen, d_eslot, n_ent, s));
            lin = Linear();
            lin.A = g->td; lin.lda = C; lin.B = L.ro; lin.ldb = C; lin.C = g->y2; lin.ldc = W; lin.M = M; lin.N = W; lin.K = C;
            ZG_TRY(launch_linear(lin, f32, s));
            if (canon && single && d.ff != ZG_LM_FF_NONE)  // the branches' mean, the residual sum, the next norm and its convolution at once
                ZG_TRY(launch_norm_conv_single(g->x, nullptr, g->y, g->y2, L.left_out, L.right_out, L.norm1b, L.norm2, eps, M, W, g->canon, L.canon2,
                                               g->seq_state + ps.canon2_off, g->seq_floats, d_slot, g->hc, s, &mid_done));
            if (!mid_done) ZG_TRY(launch_pair_norm_mean(g->y, g->y2, L.left_out, L.right_out, eps, g->y, M, W, s));
        } else if (d.mixer == ZG_LM_MIX_CHANNEL_DELTA) {
            const int G = d.kv_heads, HV = H * Vd, CC = 2 * G * D + HV, RA = d.decay_rank, RG = d.gate_rank, NP = L.n_cat;
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.wcat; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            ConvArgs cv;
            cv.in = g->proj; cv.ld_in = NP; cv.out = g->ta; cv.ld_out = CC; cv.C = CC; cv.taps = d.conv; cv.w = L.convw; cv.flags = CONV_SILU;
            cv.tail = g->seq_state + ps.conv_off; cv.slot_stride = g->seq_floats;
            ZG_TRY(launch_causal_conv(cv, M, n_ent, single, d_off, d_slot, d_estart, d_elen, d_eslot, s));
            lin = Linear();  // the decay's second step
            lin.A = g->proj + CC + H; lin.lda = NP; lin.B = L.a2; lin.ldb = RA; lin.C = g->tb; lin.ldc = H * D; lin.M = M; lin.N = H * D; lin.K = RA;
            ZG_TRY(launch_linear(lin, f32, s));
            lin = Linear();  // the output gate's second step
            lin.A = g->proj + CC + H + RA; lin.lda = NP; lin.B = L.g2; lin.ldb = RG; lin.C = g->tc; lin.ldc = HV; lin.M = M; lin.N = HV; lin.K = RG;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(launch_delta_prep(g->ta, CC, G, D, g->proj + CC, NP, H, g->tb, H * D, L.a_log, L.dt_bias, M, s));
            ZG_TRY(launch_delta_scan(g->ta, CC, g->ta + 2 * G * D, CC, g->proj + CC, NP, g->tb, H * D, g->td, HV, H, G, D, Vd,
                                     g->seq_state + ps.rec_off, g->seq_floats, d_estart, d_elen, d_eslot, n_ent, s));
            ZG_TRY(launch_norm_gate(g->td, HV, H, Vd, M, L.hnorm, eps, g->tc, HV, s));
            lin = Linear();
            lin.A = g->td; lin.lda = HV; lin.B = L.o; lin.ldb = HV; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HV;
            ZG_TRY(launch_linear(lin, f32, s));
        } else if (d.mixer == ZG_LM_MIX_GLA) {
            const int HD = H * D, HV = H * Vd, RA = d.decay_rank, NP = L.n_cat;
            const int og = 2 * HD + HV, oa = og + HV;  // columns of the output gate and of the decay's first step
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.wcat; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            lin = Linear();  // the decay's second step
            lin.A = g->proj + oa; lin.lda = NP; lin.B = L.a2; lin.ldb = RA; lin.C = g->tb; lin.ldc = HD; lin.M = M; lin.N = HD; lin.K = RA;
            ZG_TRY(launch_linear(lin, f32, s));
            GlaGate gate;
            gate.z = g->tb; gate.ldz = HD; gate.z_bias = L.a2b; gate.inv_tau = 1.0f / d.tau; gate.q_scale = 1.0f / sqrtf((float)D);
            ZG_TRY(launch_hgrn2_scan(g->proj, NP, g->o, HV, g->seq_state + ps.rec_off, g->seq_floats, d_estart, d_elen, d_eslot, n_ent, M, H, D, Vd,
                                     nullptr, nullptr, g->scan_ws, g->scan_ws_floats, s, nullptr, &gate));
            ZG_TRY(launch_norm_gate(g->o, HV, H, Vd, M, L.hnorm, eps, g->proj + og, NP, s, 1.0f, true));
            lin = Linear();
            lin.A = g->o; lin.lda = HV; lin.B = L.o; lin.ldb = HV; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HV;
            ZG_TRY(launch_linear(lin, f32, s));
        } else if (d.mixer == ZG_LM_MIX_ATTENTION) {
            const int G = d.kv_heads, HD = H * D, NP = L.n_cat;
            ScoreShape shape;
            shape.cap = d.softcap;
            shape.slope = d.dist_bias ? L.slopes : nullptr;
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.wcat; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(launch_head_norm_prep(g->proj, NP, M, H, G, D, eps, d.qtemp_coef, d.qtemp_every, d_pos, d_slot, g->page_table, g->max_pages, g->P,
                                         ps.cache, s));
            // rows of the score workspace: as long as the longest sequence of this portion (a captured decode step replays at any
            // length, so it takes the cache's capacity)
            const int all_keys = g->max_pages * g->P;
            const int key_cap = (single || capturing) ? (g->bucket_keys > 0 ? g->bucket_keys : all_keys) : std::min(all_keys, (g->step_keys + 63) / 64 * 64);
            bool split = false;
            ZG_TRY(launch_window_attention_split(g->proj, NP, g->o, HD, M, H, G, D, D, d.scale, 0, 0, nullptr, nullptr, nullptr, d_pos, d_slot,
                                                 g->page_table, g->max_pages, g->P, ps.cache, key_cap, g->win_ws, g->win_ws_floats, d_estart, d_elen,
                                                 n_ent, s, &split, nullptr, 0, 1.0f, shape));
            if (!split)
                ZG_TRY(launch_window_attention(g->proj, NP, g->o, HD, M, H, G, D, D, d.scale, 0, 0, nullptr, nullptr, nullptr, d_pos, d_slot,
                                               g->page_table, g->max_pages, g->P, ps.cache, s, shape));
            lin = Linear();
            lin.A = g->o; lin.lda = HD; lin.B = L.o; lin.ldb = HD; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HD;
            ZG_TRY(launch_linear(lin, f32, s));
        } else if (d.mixer == ZG_LM_MIX_HGRN2) {
            const int HD = H * D, HV = H * Vd, NP = 2 * HD + HV;
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.qfv; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(launch_hgrn2_scan(g->proj, NP, g->o, HV, g->hgrn_state + ps.hgrn_off, g->hgrn_floats, d_estart, d_elen, d_eslot, n_ent, M, H, D, Vd,
                                     L.fb, L.lower, g->scan_ws, g->scan_ws_floats, s));
            ZG_TRY(launch_norm_plain(g->o, HV, H, Vd, M, L.hnorm, eps, s));
            lin = Linear();
            lin.A = g->o; lin.lda = HV; lin.B = L.o; lin.ldb = HV; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HV;
            ZG_TRY(launch_linear(lin, f32, s));
        } else {
            const int R = d.rot_dim, KR = d.kv_rank, QR = d.q_rank, HV = H * Vd, NP = QR + KR + R;
            const Rotary rot{L.rot_freq, d.rot_dims, L.rot_amp};
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.dqkv; lin.ldb = W; lin.C = g->proj; lin.ldc = NP; lin.M = M; lin.N = NP; lin.K = W;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(launch_latent_prep(g->proj, NP, M, QR, KR, R, L.dq_norm, L.dkv_norm, eps, rot, d_pos, d_slot, g->page_table, g->max_pages, g->P,
                                      g->cq, ps.cache, s));
            lin = Linear();
            lin.A = g->cq; lin.lda = QR; lin.B = L.uq; lin.ldb = QR; lin.C = g->q; lin.ldc = H * (D + R); lin.M = M; lin.N = H * (D + R); lin.K = QR;
            ZG_TRY(launch_linear(lin, f32, s));
            lin = Linear();  // the unrotated query part carried into the latent space, head by head
            lin.A = g->q; lin.lda = H * (D + R); lin.a_zoff = D + R; lin.B = L.ukT; lin.ldb = D; lin.b_zoff = (long long)KR * D;
            lin.C = g->qa; lin.ldc = H * (KR + R); lin.c_zoff = KR + R; lin.M = M; lin.N = KR; lin.K = D; lin.nz = H;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(launch_q_rotary(g->q, H * (D + R), g->qa, H * (KR + R), M, H, D, R, KR, rot, d_pos, s));
            bool tiled = false;
            if (!f32 && !few)
                ZG_TRY(launch_latent_attention_tiles(g->qa, g->ctx, M, H, KR, R, d.scale, d_estart, d_elen, d_eslot, n_ent, d_pos, g->page_table,
                                                     g->max_pages, g->P, ps.cache, s, &tiled));
            if (!tiled)
                ZG_TRY(launch_latent_attention(g->qa, g->ctx, M, H, KR, R, d.scale, d_pos, d_slot, g->page_table, g->max_pages, g->P, ps.cache,
                                               g->attn_ws, g->attn_ws_floats, s));
            lin = Linear();  // values of the weighted latent, head by head
            lin.A = g->ctx; lin.lda = H * KR; lin.a_zoff = KR; lin.B = L.uv; lin.ldb = KR; lin.b_zoff = (long long)Vd * KR;
            lin.C = g->o; lin.ldc = HV; lin.c_zoff = Vd; lin.M = M; lin.N = Vd; lin.K = KR; lin.nz = H;
            ZG_TRY(launch_linear(lin, f32, s));
            lin = Linear();
            lin.A = g->o; lin.lda = HV; lin.B = L.o; lin.ldb = HV; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = HV;
            ZG_TRY(launch_linear(lin, f32, s));
        }
        if (tnorm) {  // norms without statistics: every sum behind a sublayer carries the next sublayer's norm
            const float* next_norm = p + 1 < g->n_passes ? g->layers[g->passes[p + 1].layer].norm1 : nullptr;
            SumParts part;
            part.a = g->y;
            // steps of few rows: the router's workgroups do the sum and the norms in front of them themselves
            RoutePre pre;
            const bool pre_routed = few && d.ff == ZG_LM_FF_MOE && W <= kRouteFuseWidth;
            if (pre_routed) {
                pre.x = g->x; pre.y = part; pre.nb = L.norm1b; pre.mult = g->res_mult; pre.nn = L.norm2; pre.h = g->h;
            } else {
                ZG_TRY(launch_tanh_sum_norm(g->x, part, L.norm1b, g->res_mult, d.ff != ZG_LM_FF_NONE ? L.norm2 : next_norm, g->h, M, W, s));
            }
            const int F = d.ff_width;
            part = SumParts();
            if (d.ff == ZG_LM_FF_DENSE) {
                lin = Linear();
                lin.A = g->h; lin.lda = W; lin.B = L.up; lin.ldb = W; lin.C = g->u; lin.ldc = F; lin.M = M; lin.N = F; lin.K = W; lin.act = ACT_RELU2;
                ZG_TRY(launch_linear(lin, f32, s));
                lin = Linear();
                lin.A = g->u; lin.lda = F; lin.B = L.down; lin.ldb = F; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = F;
                ZG_TRY(launch_linear(lin, f32, s));
                part.a = g->y;
            } else if (d.ff == ZG_LM_FF_MOE) {
                const int E = d.experts, top = d.top, NA = M * top;
                const bool glu = d.ff_act == ZG_LM_ACT_GLU_SILU;
                const int UF = glu ? 2 * F : F;
                ZG_TRY(launch_route(g->h, M, W, L.router, L.correction, E, top, g->pick, g->wt, d.router, s, d.route_groups, d.route_keep,
                                    d.route_scale != 0.0f ? d.route_scale : 1.0f, pre_routed ? &pre : nullptr));
                Linear up, dn;
                up.A = g->h; up.lda = W; up.a_div = top; up.B = L.gu; up.ldb = W; up.b_zoff = (long long)UF * W; up.C = g->gu_buf; up.ldc = UF;
                up.N = UF; up.K = W;
                if (!glu) up.act = ACT_GELU_ERF;
                dn.A = g->hb; dn.lda = F; dn.B = L.edown; dn.ldb = F; dn.b_zoff = (long long)W * F; dn.C = g->ye; dn.ldc = W; dn.N = W; dn.K = F;
                if (few) {  // one batch per assignment, its expert's matrices looked up on the device
                    up.M = dn.M = 1; up.nz = dn.nz = NA; up.z_group = dn.z_group = g->pick;
                    up.c_zoff = UF; dn.c_zoff = W;
                } else {  // assignments sorted by expert, grouped products
                    ZG_TRY(launch_group(g->pick, NA, E, g->grp_off, g->sorted, g->inv, s));
                    up.M = dn.M = NA; up.a_rows = g->sorted; up.grp_off = dn.grp_off = g->grp_off; up.n_groups = dn.n_groups = E;
                }
                part.exp = g->ye; part.exp_w = g->wt; part.inv = few ? nullptr : g->inv; part.top = top;
                if (few && glu && d.shared_width > 0) {
                    // steps of few rows: the expert every token uses rides in the launches of the chosen experts, a batch per row; the
                    // gated activation is applied where the second products read their rows
                    const int S = d.shared_width;
                    Linear sup, sdn;
                    sup.A = g->h; sup.lda = W; sup.a_zoff = W; sup.B = L.sgu; sup.ldb = W; sup.C = g->tb; sup.ldc = 2 * S; sup.c_zoff = 2 * S;
                    sup.M = 1; sup.nz = M; sup.N = 2 * S; sup.K = W;
                    ZG_TRY(launch_linear_pair(up, sup, f32, s));
                    dn.A = g->gu_buf; dn.lda = 2 * F; dn.a_glu = F;
                    sdn.A = g->tb; sdn.lda = 2 * S; sdn.a_zoff = 2 * S; sdn.a_glu = S; sdn.B = L.sdown; sdn.ldb = S; sdn.C = g->td; sdn.ldc = W;
                    sdn.c_zoff = W; sdn.M = 1; sdn.nz = M; sdn.N = W; sdn.K = S;
                    ZG_TRY(launch_linear_pair(dn, sdn, f32, s));
                    part.b = g->td;
                    ZG_TRY(launch_tanh_sum_norm(g->x, part, L.norm2b, g->res_mult, next_norm, g->h, M, W, s));
                    h_ready = next_norm != nullptr;
                    ZG_TRY(copy_trace(p));
                    continue;
                }
                ZG_TRY(launch_linear(up, f32, s));
                if (!glu) {  // the first product's epilogue has applied the activation
                    dn.A = g->gu_buf; dn.lda = F;
                } else if (few) {  // the gated activation is applied where the second product reads its rows
                    dn.A = g->gu_buf; dn.lda = 2 * F; dn.a_glu = F;
                } else {
                    ZG_TRY(launch_glu(g->gu_buf, g->hb, NA, F, s));
                }
                ZG_TRY(launch_linear(dn, f32, s));
                if (d.shared_width > 0) {  // the expert every token uses
                    const int S = d.shared_width;
                    lin = Linear();
                    lin.A = g->h; lin.lda = W; lin.B = L.sgu; lin.ldb = W; lin.C = g->tb; lin.ldc = 2 * S; lin.M = M; lin.N = 2 * S; lin.K = W;
                    ZG_TRY(launch_linear(lin, f32, s));
                    lin = Linear();
                    lin.B = L.sdown; lin.ldb = S; lin.C = g->td; lin.ldc = W; lin.M = M; lin.N = W; lin.K = S;
                    if (M <= 2) {  // the activation where the second product reads its rows (more rows: every workgroup would redo it)
                        lin.A = g->tb; lin.lda = 2 * S; lin.a_glu = S;
                    } else {
                        ZG_TRY(launch_glu(g->tb, g->tc, M, S, s));
                        lin.A = g->tc; lin.lda = S;
                    }
                    ZG_TRY(launch_linear(lin, f32, s));
                    part.b = g->td;
                }
            }
            if (d.ff != ZG_LM_FF_NONE) ZG_TRY(launch_tanh_sum_norm(g->x, part, L.norm2b, g->res_mult, next_norm, g->h, M, W, s));
            h_ready = next_norm != nullptr;
            ZG_TRY(copy_trace(p));
            continue;
        }
        if (side) {  // the feed-forward beside the mixer, on the second norm of the same x
            const int F = d.ff_width;
            const float* fin = g->hc;
            if (d.ff == ZG_LM_FF_DENSE) {
                lin = Linear();
                lin.A = fin; lin.lda = W; lin.B = L.up; lin.ldb = W; lin.C = g->u; lin.ldc = F; lin.M = M; lin.N = F; lin.K = W; lin.act = ACT_RELU2;
                ZG_TRY(launch_linear(lin, f32, s));
                lin = Linear();
                lin.A = g->u; lin.lda = F; lin.B = L.down; lin.ldb = F; lin.C = g->y2; lin.ldc = W; lin.M = M; lin.N = W; lin.K = F;
                ZG_TRY(launch_linear(lin, f32, s));
            } else if (d.ff == ZG_LM_FF_MOE) {
                const int E = d.experts, top = d.top, NA = M * top;
                const int UF = d.ff_act == ZG_LM_ACT_GELU ? F : 2 * F;
                const bool on_input = d.router == ZG_LM_ROUTE_SIGMOID_INPUT;  // the router's score multiplies the expert's input
                ZG_TRY(launch_route(fin, M, W, L.router, L.correction, E, top, g->pick, g->wt, d.router, s, d.route_groups, d.route_keep,
                                    d.route_scale != 0.0f ? d.route_scale : 1.0f));
                Linear up, dn;
                up.A = fin; up.lda = W; up.a_div = top; up.B = L.gu; up.ldb = W; up.b_zoff = (long long)UF * W; up.C = g->gu_buf; up.ldc = UF;
                up.N = UF; up.K = W;
                if (d.ff_act == ZG_LM_ACT_GELU) up.act = ACT_GELU_ERF;
                dn.A = g->hb; dn.lda = F; dn.B = L.edown; dn.ldb = F; dn.b_zoff = (long long)W * F; dn.C = g->ye; dn.ldc = W; dn.N = W; dn.K = F;
                if (few) {  // one batch per assignment, its expert's matrices looked up on the device
                    up.M = dn.M = 1; up.nz = dn.nz = NA; up.z_group = dn.z_group = g->pick;
                    up.c_zoff = UF; dn.c_zoff = W;
                } else {  // assignments sorted by expert, grouped products
                    ZG_TRY(launch_group(g->pick, NA, E, g->grp_off, g->sorted, g->inv, s));
                    up.M = dn.M = NA; up.a_rows = g->sorted; up.grp_off = dn.grp_off = g->grp_off; up.n_groups = dn.n_groups = E;
                }
                ZG_TRY(launch_linear(up, f32, s));
                // (the product is linear: the score that multiplies an expert's input is applied to the product, in front of the clip)
                if (d.ff_act == ZG_LM_ACT_GELU) {
                    dn.A = g->gu_buf; dn.lda = F;
                } else if (d.ff_act == ZG_LM_ACT_GLU_SILU) {
                    ZG_TRY(launch_glu(g->gu_buf, g->hb, NA, F, s));
                } else if (few) {  // the activation is applied where the second product reads its rows
                    dn.A = g->gu_buf; dn.lda = 2 * F; dn.a_glu = F; dn.glu_kind = GLU_CLIPPED; dn.glu_limit = d.ff_limit;
                    dn.glu_scale = on_input ? g->wt : nullptr;
                } else {
                    ZG_TRY(launch_glu_clipped(g->gu_buf, UF, g->hb, NA, F, d.ff_limit, on_input ? g->wt : nullptr, g->sorted, -1, s));
                }
                ZG_TRY(launch_linear(dn, f32, s));
                const float* ys = nullptr;
                if (d.shared_width > 0) {  // the shared expert; its gate logit is the last column of its first product
                    const int S = d.shared_width;
                    lin = Linear();
                    lin.A = fin; lin.lda = W; lin.B = L.sgu; lin.ldb = W; lin.C = g->tb; lin.ldc = 2 * S + 1; lin.M = M; lin.N = 2 * S + 1; lin.K = W;
                    ZG_TRY(launch_linear(lin, f32, s));
                    lin = Linear();
                    lin.B = L.sdown; lin.ldb = S; lin.C = g->td; lin.ldc = W; lin.M = M; lin.N = W; lin.K = S;
                    if (M <= 2) {  // activation and gate where the second product reads its rows (more rows: every workgroup would redo them)
                        lin.A = g->tb; lin.lda = 2 * S + 1; lin.a_glu = S; lin.glu_kind = GLU_CLIPPED; lin.glu_limit = d.shared_limit; lin.glu_gate_col = 2 * S;
                    } else {
                        ZG_TRY(launch_glu_clipped(g->tb, 2 * S + 1, g->tc, M, S, d.shared_limit, nullptr, nullptr, 2 * S, s));
                        lin.A = g->tc; lin.lda = S;
                    }
                    ZG_TRY(launch_linear(lin, f32, s));
                    ys = g->td;
                }
                if (few) {  // the experts' rows are added where the open sums are
                    pend.exp = g->ye;
                    pend.exp_w = on_input ? nullptr : g->wt;
                    pend.top = top;
                    pend.b = ys;
                } else {
                    ZG_TRY(launch_expert_sum(g->y2, g->ye, g->inv, on_input ? nullptr : g->wt, top, ys, M, W, s));
                    pend.b = g->y2;
                }
            }
            pend.a = g->y;
            if (d.ff == ZG_LM_FF_DENSE) pend.b = g->y2;
            pend.bias = d.mixer == ZG_LM_MIX_WINDOW_LINEAR ? L.obias : nullptr;
            pend.w = d.left_scale;
            if (p + 1 == g->n_passes || (g->trace && !capturing)) {  // nobody behind to add them (or the stream is to be shown): add now
                ZG_TRY(launch_add_two(g->x, pend, M, W, s));
                pend = OpenSums();
            }
            ZG_TRY(copy_trace(p));
            h_ready = false;
            continue;
        }
        if (canon && single && d.ff != ZG_LM_FF_NONE && !mid_done)
            ZG_TRY(launch_norm_conv_single(g->x, nullptr, g->y, nullptr, nullptr, nullptr, L.norm1b, L.norm2, eps, M, W, g->canon, L.canon2,
                                           g->seq_state + ps.canon2_off, g->seq_floats, d_slot, g->hc, s, &mid_done));
        if (mid_done) {
        } else if (d.ff != ZG_LM_FF_NONE) ZG_TRY(launch_norm_add_norm(g->x, g->y, L.norm1b, L.norm2, eps, g->h, M, W, s));
        else {
            ZG_TRY(tail(g->y, nullptr, nullptr, 0, L.norm1b));
            if (!h_ready) ZG_TRY(launch_norm_add(g->x, g->y, L.norm1b, eps, M, W, s));
        }
        const int F = d.ff_width;
        hin = g->h;
        if (canon && d.ff != ZG_LM_FF_NONE) {
            if (!mid_done) ZG_TRY(input_conv(L.canon2, ps.canon2_off));
            hin = g->hc;
        }
        if (d.ff == ZG_LM_FF_DENSE) {
            lin = Linear();
            lin.A = hin; lin.lda = W; lin.B = L.up; lin.ldb = W; lin.C = g->u; lin.ldc = F; lin.M = M; lin.N = F; lin.K = W; lin.act = ACT_RELU2;
            ZG_TRY(launch_linear(lin, f32, s));
            lin = Linear();
            lin.A = g->u; lin.lda = F; lin.B = L.down; lin.ldb = F; lin.C = g->y; lin.ldc = W; lin.M = M; lin.N = W; lin.K = F;
            ZG_TRY(launch_linear(lin, f32, s));
            ZG_TRY(tail(g->y, nullptr, nullptr, 0, L.norm2b));
            if (!h_ready) ZG_TRY(launch_norm_add(g->x, g->y, L.norm2b, eps, M, W, s));
        } else if (d.ff == ZG_LM_FF_MOE) {
            const int E = d.experts, top = d.top, NA = M * top;
            const bool glu = d.ff_act == ZG_LM_ACT_GLU_SILU;
            const int UF = glu ? 2 * F : F;
            ZG_TRY(launch_route(hin, M, W, L.router, L.correction, E, top, g->pick, g->wt, d.router, s, d.route_groups, d.route_keep,
                                d.route_scale != 0.0f ? d.route_scale : 1.0f));
            Linear up, dn;
            up.A = hin; up.lda = W; up.a_div = top; up.B = L.gu; up.ldb = W; up.b_zoff = (long long)UF * W; up.C = g->gu_buf; up.ldc = UF;
            up.N = UF; up.K = W;
            if (!glu) up.act = ACT_GELU_ERF;
            dn.A = g->hb; dn.lda = F; dn.B = L.edown; dn.ldb = F; dn.b_zoff = (long long)W * F; dn.C = g->ye; dn.ldc = W; dn.N = W; dn.K = F;
            if (few) {  // one batch per assignment, its expert's matrices looked up on the device
                up.M = dn.M = 1; up.nz = dn.nz = NA; up.z_group = dn.z_group = g->pick;
                up.c_zoff = UF; dn.c_zoff = W;
            } else {  // assignments sorted by expert, grouped products
                ZG_TRY(launch_group(g->pick, NA, E, g->grp_off, g->sorted, g->inv, s));
                up.M = dn.M = NA; up.a_rows = g->sorted; up.grp_off = dn.grp_off = g->grp_off; up.n_groups = dn.n_groups = E;
            }
            ZG_TRY(launch_linear(up, f32, s));
            if (!glu) {  // the first product's epilogue has applied the activation
                dn.A = g->gu_buf; dn.lda = F;
            } else if (few) {  // the gated activation is applied where the second product reads its rows
                dn.A = g->gu_buf; dn.lda = 2 * F; dn.a_glu = F;
            } else {
                ZG_TRY(launch_glu(g->gu_buf, g->hb, NA, F, s));
            }
            ZG_TRY(launch_linear(dn, f32, s));
            if (few) ZG_TRY(tail(nullptr, g->ye, g->wt, top, L.norm2b));
            if (!h_ready) ZG_TRY(launch_moe_combine(g->x, g->ye, few ? nullptr : g->inv, g->wt, top, L.norm2b, eps, M, W, s));
        }
        ZG_TRY(copy_trace(p));
    }
    // the rows the last tokens of the entries left for the token shift of their successors
    if (!canon && !side && !tnorm) ZG_TRY(launch_commit_rows(g->shift_state, (size_t)g->n_passes * W, g->last_h, W, d_eslot, n_ent, W, g->n_passes, W, (size_t)NS * W, s));

    return ZG_OK;
}

// ------------------------------------------------------------------------------------------------ one portion of rows
int run_portion(zg_lm* g, const std::vector<Piece>& pieces, float* logits_out, const Sampler* sampler) {
    hipStream_t s = g->stream;
    const int W = g->W, MS = g->MS, NS = g->NS;
    int M = 0;
    for (const Piece& pc : pieces) M += pc.n;
    if (M == 0) return ZG_OK;
    const int n_ent = (int)pieces.size();
    int *ids = g->h_meta, *pos = ids + MS, *slot = pos + MS, *prev = slot + MS, *lastent = prev + MS, *want_rows = lastent + MS;
    int *ent_start = want_rows + MS, *ent_len = ent_start + NS, *ent_slot = ent_len + NS;
    int* row_off = g->h_meta + meta_row_off(g);
    std::vector<std::pair<int, size_t>> wants;  // (row of the portion, output row)
    int r = 0;
    g->step_keys = 0;
    for (int e = 0; e < n_ent; ++e) {
        const Piece& pc = pieces[e];
        g->step_keys = std::max(g->step_keys, pc.pos0 + pc.n);
        ent_start[e] = r;
        ent_len[e] = pc.n;
        ent_slot[e] = pc.slot;
        for (int t = 0; t < pc.n; ++t, ++r) {
            ids[r] = pc.tok[t];
            pos[r] = pc.pos0 + t;
            slot[r] = pc.slot;
            prev[r] = t > 0 ? r - 1 : -1;
            lastent[r] = t == pc.n - 1 ? e : -1;
            row_off[r] = t;
        }
        for (auto& w : pc.wants) wants.push_back({ent_start[e] + w.first, w.second});
        const Slot& sl = g->slots[pc.slot];
        ZG_HIP(hipMemcpyAsync(g->page_table + (size_t)pc.slot * g->max_pages, sl.ring.data(), sl.ring.size() * sizeof(int), hipMemcpyHostToDevice, s));
    }
    ZG_HIP(hipMemcpyAsync(g->meta, g->h_meta, meta_ints(g) * sizeof(int), hipMemcpyHostToDevice, s));
    const int* d_want = g->meta + 5 * (size_t)MS;
    const bool f32 = g->f32;
    const float eps = g->cfg.norm_eps;

    ZG_HIP(hipEventRecord(g->ev0, s));
    bool single = M <= kGemvMaxRows && !g->trace && g->use_graph;
    for (const Piece& pc : pieces) single = single && pc.n == 1;
    int bucket = 0;
    g->bucket_keys = 0;
    if (g->whole_context) {  // the smallest bucket that holds the longest sequence of the step
        const int all_keys = g->max_pages * g->P;
        while (bucket + 1 < zg_lm::kKeyBuckets && (512LL << bucket) < g->step_keys) ++bucket;
        g->bucket_keys = (int)std::min<long long>(all_keys, 512LL << bucket);
    }
    if (single) {  // a decode step: replay the captured sequence of this batch size
        if (!g->decode_graph[M][bucket]) {
            hipGraph_t graph = nullptr;
            ZG_HIP(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal));
            const int st = enqueue_layers(g, M, n_ent, true, true);
            const hipError_t ce = hipStreamEndCapture(s, &graph);
            if (st != ZG_OK) {
                if (graph) (void)hipGraphDestroy(graph);
                return st;
            }
            ZG_HIP(ce);
            ZG_HIP(hipGraphInstantiate(&g->decode_graph[M][bucket], graph, nullptr, nullptr, 0));
            ZG_HIP(hipGraphDestroy(graph));
        }
        ZG_HIP(hipGraphLaunch(g->decode_graph[M][bucket], s));
    } else {
        bool one_row = M <= kGemvMaxRows;
        for (const Piece& pc : pieces) one_row = one_row && pc.n == 1;
        ZG_TRY(enqueue_layers(g, M, n_ent, false, one_row));
    }

    // logits of the rows that were asked for, logit_rows at a time
    size_t w0 = 0;
    do {
        const int nw = (int)std::min<size_t>(g->logit_rows, wants.size() - w0);
        if (nw > 0) {
            // (the want rows travel through the pinned twin of the metadata; the stream is drained at the end of every batch,
            // so the twin is free again when the next batch fills it)
            for (int j = 0; j < nw; ++j) want_rows[j] = wants[w0 + j].first;
            ZG_HIP(hipMemcpyAsync(g->meta + 5 * (size_t)MS, want_rows, nw * sizeof(int), hipMemcpyHostToDevice, s));
            if (g->tanh_norms) ZG_TRY(launch_tanh_norm(g->x, nullptr, g->final_norm, d_want, g->hn, nw, W, s));
            else ZG_TRY(launch_norm_gather(g->x, d_want, g->final_norm, eps, g->hn, nw, W, g->side, s));
            Linear lin;
            lin.A = g->hn; lin.lda = W; lin.B = g->head; lin.ldb = W; lin.C = g->logits; lin.ldc = g->V; lin.M = nw; lin.N = g->V; lin.K = W;
            if ((g->cfg.logit_scale != 0.0f && g->cfg.logit_scale != 1.0f) || g->cfg.logit_softcap > 0.0f) {
                lin.act = ACT_SCALE_SOFTCAP;
                lin.act_a = g->cfg.logit_scale != 0.0f ? g->cfg.logit_scale : 1.0f;
                lin.act_b = g->cfg.logit_softcap;
            }
            ZG_TRY(launch_linear(lin, f32, s));
            if (sampler) {
                ZG_TRY(launch_row_argmax(g->logits, nw, g->V, g->row_max, g->tok_out, g->amax_val, g->amax_idx, s));
                if (sampler->temp > 0.0f) {
                    for (int j = 0; j < nw; ++j) {  // the uniform of (seed, length of the sequence with the token to be drawn, output row)
                        const int row = wants[w0 + j].first;
                        uint64_t z = sampler->seed * 0x9E3779B97F4A7C15ULL + (uint64_t)(pos[row] + 2) * 0xD1B54A32D192ED03ULL + wants[w0 + j].second + 1;
                        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
                        z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
                        z ^= z >> 31;
                        g->h_u[j] = (float)(uint32_t)(z >> 40) * 5.9604644775390625e-08f;
                    }
                    ZG_HIP(hipMemcpyAsync(g->samp_u, g->h_u, nw * sizeof(float), hipMemcpyHostToDevice, s));
                    ZG_TRY(launch_sample(g->logits, nw, g->V, sampler->temp, g->samp_u, g->row_max, 1, 1, g->samp_ws, g->tok_out, false, s));
                }
                ZG_HIP(hipMemcpyAsync(g->h_small, g->tok_out, nw * sizeof(int), hipMemcpyDeviceToHost, s));
            } else if (logits_out) {
                ZG_HIP(hipMemcpyAsync(g->h_logits, g->logits, (size_t)nw * g->V * sizeof(float), hipMemcpyDeviceToHost, s));
            }
        }
        if (w0 + nw >= wants.size()) ZG_HIP(hipEventRecord(g->ev1, s));
        ZG_HIP(hipMemcpyAsync(g->h_small + g->logit_rows, g->flag, sizeof(int), hipMemcpyDeviceToHost, s));
        ZG_HIP(hipStreamSynchronize(s));
        for (int j = 0; j < nw; ++j) {
            const size_t out_row = wants[w0 + j].second;
            if (sampler) sampler->tokens_out[out_row] = g->h_small[j];
            else if (logits_out) memcpy(logits_out + out_row * g->V, g->h_logits + (size_t)j * g->V, (size_t)g->V * sizeof(float));
        }
        w0 += nw;
    } while (w0 < wants.size());
    float ms = 0.0f;
    ZG_HIP(hipEventElapsedTime(&ms, g->ev0, g->ev1));
    g->last_step_ms += ms;
    ZG_REQUIRE(g->h_small[g->logit_rows] == 0, ZG_ERR_ARG, "step: a token id outside the vocabulary of %d", g->V);
    return ZG_OK;
}

int step_impl(zg_lm* g, const zg_lm_entry* entries, size_t n_entries, float* logits_out, size_t logits_len, const Sampler* sampler) {
    ZG_REQUIRE(g && (entries || n_entries == 0), ZG_ERR_ARG, "lm_step: bad argument");
    ZG_HIP(hipSetDevice(g->device));
    size_t n_want = 0, need_pages = 0;
    for (size_t i = 0; i < n_entries; ++i) {
        const zg_lm_entry& e = entries[i];
        ZG_REQUIRE(e.seq >= 0 && e.seq < g->NS && g->slots[e.seq].open, ZG_ERR_ARG, "lm_step: entry %zu names sequence %d, which is not open", i, e.seq);
        for (size_t j = 0; j < i; ++j) ZG_REQUIRE(entries[j].seq != e.seq, ZG_ERR_ARG, "lm_step: sequence %d appears in two entries", e.seq);
        ZG_REQUIRE(e.n_tokens == 0 || e.tokens, ZG_ERR_ARG, "lm_step: entry %zu has no tokens", i);
        ZG_REQUIRE(e.n_want == 0 || e.want, ZG_ERR_ARG, "lm_step: entry %zu has no want list", i);
        for (size_t t = 0; t < e.n_tokens; ++t)
            ZG_REQUIRE(e.tokens[t] >= 0 && e.tokens[t] < g->V, ZG_ERR_ARG, "lm_step: token %d outside the vocabulary of %d", e.tokens[t], g->V);
        for (size_t j = 0; j < e.n_want; ++j)
            ZG_REQUIRE(e.want[j] >= 0 && (size_t)e.want[j] < e.n_tokens, ZG_ERR_ARG, "lm_step: entry %zu asks for place %d of %zu tokens", i, e.want[j],
                       e.n_tokens);
        n_want += e.n_want;
        const Slot& sl = g->slots[e.seq];
        const size_t pages = (sl.len + e.n_tokens + g->P - 1) / g->P;
        ZG_REQUIRE(pages - sl.first_live <= (size_t)g->max_pages, ZG_ERR_SHAPE, "lm_step: sequence %d would hold %zu tokens in the cache (at most %zu)",
                   e.seq, sl.len + e.n_tokens - sl.first_live * g->P, (size_t)g->max_pages * g->P);
        need_pages += pages > sl.pages.size() ? pages - sl.pages.size() : 0;
    }
    ZG_REQUIRE(need_pages <= g->free_pages.size(), ZG_ERR_SHAPE, "lm_step: %zu cache pages needed, %zu free (max_tokens %zu)", need_pages,
               g->free_pages.size(), g->cfg.max_tokens);
    ZG_REQUIRE(sampler || n_want == 0 || (logits_out && logits_len >= n_want * (size_t)g->V), ZG_ERR_SHAPE, "lm_step: logits_out needs %zu elements",
               n_want * (size_t)g->V);
    for (size_t i = 0; i < n_entries; ++i) {
        Slot& sl = g->slots[entries[i].seq];
        const size_t pages = (sl.len + entries[i].n_tokens + g->P - 1) / g->P;
        while (sl.pages.size() < pages) {
            sl.ring[sl.pages.size() % g->max_pages] = g->free_pages.back();
            sl.pages.push_back(g->free_pages.back());
            g->free_pages.pop_back();
        }
    }
    g->last_step_ms = 0.0f;
    // cut the entries into portions of at most max_step_tokens rows
    std::vector<Piece> pieces;
    int rows = 0;
    size_t out_base = 0;
    for (size_t i = 0; i < n_entries; ++i) {
        const zg_lm_entry& e = entries[i];
        Slot& sl = g->slots[e.seq];
        size_t done = 0;
        while (done < e.n_tokens) {
            const int n = (int)std::min<size_t>(e.n_tokens - done, (size_t)(g->MS - rows));
            Piece pc;
            pc.slot = e.seq;
            pc.tok = e.tokens + done;
            pc.n = n;
            pc.pos0 = (int)(sl.len + done);
            for (size_t j = 0; j < e.n_want; ++j)
                if ((size_t)e.want[j] >= done && (size_t)e.want[j] < done + n) pc.wants.push_back({(int)(e.want[j] - done), out_base + j});
            pieces.push_back(pc);
            rows += n;
            done += n;
            if (rows == g->MS) {
                ZG_TRY(run_portion(g, pieces, logits_out, sampler));
                pieces.clear();
                rows = 0;
            }
        }
        sl.len += e.n_tokens;
        out_base += e.n_want;
    }
    if (!pieces.empty()) ZG_TRY(run_portion(g, pieces, logits_out, sampler));
    if (g->keep_tokens > 0)  // pages whose every token lies behind the longest window return to the pool
        for (size_t i = 0; i < n_entries; ++i) {
            Slot& sl = g->slots[entries[i].seq];
            if (sl.len + 1 <= (size_t)g->keep_tokens) continue;
            const size_t dead = (sl.len + 1 - g->keep_tokens) / g->P;  // the next token sees positions >= len + 1 - keep
            for (size_t pg = g->keep_pages; pg < dead && pg < sl.pages.size(); ++pg)
                if (sl.pages[pg] >= 0) {
                    g->free_pages.push_back(sl.pages[pg]);
                    sl.pages[pg] = -1;
                }
            if (g->keep_pages == 0) sl.first_live = std::max(sl.first_live, std::min(dead, sl.pages.size()));
        }
    return ZG_OK;
}

}  // namespace

extern "C" {

int zg_lm_create(zg_lm** out, const zg_lm_config* config, int device) {
    ZG_REQUIRE(out && config && config->layers && config->n_layers >= 1, ZG_ERR_ARG, "lm_create: bad argument");
    ZG_REQUIRE(config->vocab >= 1 && config->width >= 1 && config->vocab <= 262144, ZG_ERR_ARG, "lm_create: vocab %zu width %zu", config->vocab,
               config->width);
    ZG_REQUIRE(config->norm_eps >= 0.0f, ZG_ERR_ARG, "lm_create: norm eps %g", config->norm_eps);
    int n_dev = 0;
    ZG_HIP(hipGetDeviceCount(&n_dev));
    ZG_REQUIRE(device >= 0 && device < n_dev, ZG_ERR_ARG, "device %d out of range (%d visible)", device, n_dev);
    ZG_HIP(hipSetDevice(device));
    hipDeviceProp_t prop;
    ZG_HIP(hipGetDeviceProperties(&prop, device));
    ZG_REQUIRE(strncmp(prop.gcnArchName, "gfx950", 6) == 0, ZG_ERR_UNSUPPORTED, "built for gfx950 (MI355X) only; device %d is %s", device,
               prop.gcnArchName);
    zg_lm* g = new zg_lm();
    g->cfg = *config;
    g->device = device;
    g->f32 = (config->flags & ZG_LM_F32) != 0;
    g->use_graph = (config->flags & ZG_LM_NO_GRAPH) == 0;
    g->W = (int)config->width;
    g->V = (int)config->vocab;
    g->MS = (int)(config->max_step_tokens ? config->max_step_tokens : 2048);
    g->NS = (int)std::max<size_t>(1, config->max_seqs);
    g->P = (int)(config->page_tokens ? config->page_tokens : 64);
    const size_t max_tokens = std::max<size_t>(1, config->max_tokens);
    g->max_pages = (int)((max_tokens + g->P - 1) / g->P);
    g->n_pages = g->max_pages + g->NS;  // every open sequence may leave one page partly used
    g->logit_rows = std::min(g->MS, 256);
    g->canon = config->canon_taps;
    g->side = (config->flags & ZG_LM_SIDE_BY_SIDE) != 0;
    g->tanh_norms = (config->flags & ZG_LM_TANH_NORMS) != 0;
    g->res_mult = config->residual_mult != 0.0f ? config->residual_mult : 1.0f;
    g->embed_scale = config->embed_scale != 0.0f ? config->embed_scale : 1.0f;
    int status = ZG_OK;
    for (size_t i = 0; i < config->n_layers && status == ZG_OK; ++i) {
        status = check_layer(config->layers[i], i, config->flags);
        LayerW L;
        L.d = config->layers[i];
        g->layers.push_back(L);
    }
    g->cfg.layers = nullptr;
    // a layer that runs another layer's tensors: follow the chain to the layer that owns them
    std::vector<int> owner(config->n_layers);
    for (size_t i = 0; i < config->n_layers && status == ZG_OK; ++i) {
        size_t j = i, hops = 0;
        while (g->layers[j].d.weights_of > 0 && status == ZG_OK) {
            const int w = g->layers[j].d.weights_of - 1;
            if (w < 0 || (size_t)w >= config->n_layers || (size_t)w == j || ++hops > config->n_layers) {
                set_error("lm_create: layer %zu names the weights of layer %d", j, w);
                status = ZG_ERR_ARG;
                break;
            }
            j = (size_t)w;
        }
        owner[i] = (int)j;
        if (status == ZG_OK && j != i) {
            const zg_lm_layer &a = g->layers[i].d, &o = g->layers[j].d;
            if (a.mixer != o.mixer || a.heads != o.heads || a.dim != o.dim || a.vdim != o.vdim || a.kv_heads != o.kv_heads || a.ff != o.ff ||
                a.ff_width != o.ff_width || a.experts != o.experts || a.top != o.top || a.shared_width != o.shared_width) {
                set_error("lm_create: layer %zu names the weights of layer %zu, whose sizes differ", i, j);
                status = ZG_ERR_ARG;
            }
        }
    }
    if (status == ZG_OK && g->tanh_norms && (g->side || g->canon != 0 || (config->flags & ZG_LM_LOOP_READD))) {
        set_error("lm_create: the norms without statistics stand in sequential sublayers, without input convolution or re-added embedding");
        status = ZG_ERR_UNSUPPORTED;
    }
    if (status == ZG_OK && !g->tanh_norms && (config->flags & ZG_LM_EMBED_NORM)) {
        set_error("lm_create: a norm behind the embedding is built for the norms without statistics");
        status = ZG_ERR_UNSUPPORTED;
    }
    if (status == ZG_OK && g->side && (g->canon != 0 || config->loop_times > 1)) {
        set_error("lm_create: side-by-side sublayers have no input convolution and no looped span");
        status = ZG_ERR_UNSUPPORTED;
    }
    if (status == ZG_OK && (g->canon < 0 || g->canon > 16)) {
        set_error("lm_create: %d taps of the input convolution (0 to 16)", g->canon);
        status = ZG_ERR_ARG;
    }
    const int n = (int)config->n_layers;
    int a = 0, b = 0, k = 1;
    if (status == ZG_OK && config->loop_times > 1) {
        a = config->loop_start; b = config->loop_stop; k = config->loop_times;
        if (!(a >= 0 && a <= b && b <= n)) {
            set_error("lm_create: loop [%d, %d) outside the %d layers", a, b, n);
            status = ZG_ERR_ARG;
        }
    }
    if (status != ZG_OK) {
        delete g;
        return status;
    }
    auto add = [&](int layer) {
        Pass ps;
        ps.layer = owner[layer];
        g->passes.push_back(ps);
    };
    for (int i = 0; i < a; ++i) add(i);
    for (int t = 0; t < k; ++t)
        for (int i = a; i < b; ++i) {
            add(i);
            g->passes.back().readd = t > 0 && i == a && (config->flags & ZG_LM_LOOP_READD);
        }
    for (int i = (k > 1 ? b : 0); i < n; ++i) add(i);
    g->n_passes = (int)g->passes.size();
    // how far back any attention pass looks: pages behind that are given back while a sequence is still open
    bool attends = false, bounded = true;
    for (const Pass& ps : g->passes) {
        const zg_lm_layer& d = g->layers[ps.layer].d;
        if (d.mixer == ZG_LM_MIX_LATENT_ATTENTION || d.mixer == ZG_LM_MIX_ATTENTION || (d.mixer == ZG_LM_MIX_PARALLEL && d.window == 0))
            attends = true, bounded = false;
        if (d.mixer == ZG_LM_MIX_ATTENTION) g->whole_context = true;
        if (d.mixer == ZG_LM_MIX_PARALLEL && d.window > 0) {
            attends = true;
            g->keep_tokens = std::max(g->keep_tokens, d.window);
        }
        if (d.mixer == ZG_LM_MIX_WINDOW_LINEAR) {
            attends = true;
            if (d.window > 0) {
                g->keep_tokens = std::max(g->keep_tokens, d.window);
                g->keep_first = std::max(g->keep_first, d.keep_first);
            } else {
                bounded = false;
            }
        }
    }
    if (!attends || !bounded) g->keep_tokens = 0;
    // kept first tokens hold their pages for good: the pages between them and the window go back to the pool, but the page table
    // cannot wrap round (a sequence is then bounded by the table: max_tokens)
    g->keep_pages = g->keep_tokens > 0 ? (g->keep_first + g->P - 1) / g->P : 0;
    Bump measure{nullptr};
    layout(g, measure);
    g->arena_bytes = measure.off + 256;
    auto fail = [&](int code) {
        zg_lm_destroy(g);
        return code;
    };
    if (hipMalloc(reinterpret_cast<void**>(&g->arena), g->arena_bytes) != hipSuccess) {
        (void)hipGetLastError();
        set_error("lm_create: %zu bytes of device memory not available", g->arena_bytes);
        g->arena = nullptr;
        return fail(ZG_ERR_HIP);
    }
    Bump place{g->arena};
    layout(g, place);
#define ZG_LM_TRY_HIP(expr)                                       \
    do {                                                          \
        hipError_t _e = (expr);                                   \
        if (_e != hipSuccess) return fail(hip_fail(_e, #expr, __FILE__, __LINE__)); \
    } while (0)
    ZG_LM_TRY_HIP(hipStreamCreateWithFlags(&g->stream, hipStreamNonBlocking));
    ZG_LM_TRY_HIP(hipEventCreate(&g->ev0));
    ZG_LM_TRY_HIP(hipEventCreate(&g->ev1));
    ZG_LM_TRY_HIP(hipHostMalloc(reinterpret_cast<void**>(&g->h_meta), meta_ints(g) * sizeof(int), hipHostMallocDefault));
    ZG_LM_TRY_HIP(hipHostMalloc(reinterpret_cast<void**>(&g->h_logits), (size_t)g->logit_rows * g->V * sizeof(float), hipHostMallocDefault));
    ZG_LM_TRY_HIP(hipHostMalloc(reinterpret_cast<void**>(&g->h_small), (g->logit_rows + 16) * sizeof(int), hipHostMallocDefault));
    ZG_LM_TRY_HIP(hipHostMalloc(reinterpret_cast<void**>(&g->h_u), g->logit_rows * sizeof(float), hipHostMallocDefault));
    memset(g->h_meta, 0, meta_ints(g) * sizeof(int));
    // state and flags start at zero; rotary tables
    const size_t state_floats = (size_t)g->NS * g->n_passes * g->W;
    zero_kernel<<<(unsigned)((state_floats + 255) / 256), 256, 0, g->stream>>>(g->shift_state, state_floats);
    zero_kernel<<<1, 256, 0, g->stream>>>(reinterpret_cast<float*>(g->flag), 16);
    zero_kernel<<<(unsigned)(((size_t)g->NS * g->max_pages + 255) / 256), 256, 0, g->stream>>>(reinterpret_cast<float*>(g->page_table),
                                                                                            (size_t)g->NS * g->max_pages);
    if (g->seq_floats) {
        const size_t nsq = (size_t)g->NS * g->seq_floats;
        zero_kernel<<<(unsigned)((nsq + 255) / 256), 256, 0, g->stream>>>(g->seq_state, nsq);
    }
    if (g->pos_freq) {  // 10000^(-2i/W), rounded once
        std::vector<float> pf((g->W + 1) / 2);
        for (size_t i = 0; i < pf.size(); ++i) pf[i] = (float)pow(10000.0, -2.0 * (double)i / (double)g->W);
        ZG_LM_TRY_HIP(hipMemcpy(g->pos_freq, pf.data(), pf.size() * sizeof(float), hipMemcpyHostToDevice));
    }
    for (LayerW& L : g->layers)
        if (L.d.mixer == ZG_LM_MIX_WINDOW_LINEAR && L.d.conv == 0 && L.d.weights_of == 0) {  // no convolution: one tap of weight one
            const size_t n = (size_t)L.d.heads * L.d.dim + (size_t)L.d.kv_heads * (L.d.dim + L.d.vdim);
            ones_kernel<<<(unsigned)((n + 255) / 256), 256, 0, g->stream>>>(L.convw, n);
        }
    for (LayerW& L : g->layers)
        if (L.d.mixer == ZG_LM_MIX_ATTENTION && L.slopes) {  // head h loses 2^(-8 (h + 1) / heads) per position of distance
            std::vector<float> sl(L.d.heads);
            for (int h = 0; h < L.d.heads; ++h) sl[h] = (float)pow(2.0, -8.0 * (h + 1) / (double)L.d.heads);
            ZG_LM_TRY_HIP(hipMemcpy(L.slopes, sl.data(), sl.size() * sizeof(float), hipMemcpyHostToDevice));
        }
    for (LayerW& L : g->layers)
        if ((L.d.mixer == ZG_LM_MIX_LATENT_ATTENTION || L.d.mixer == ZG_LM_MIX_PARALLEL) && L.d.weights_of == 0) {
            std::vector<float> freq;
            rotary_table(L.d, freq, L.rot_amp);
            ZG_LM_TRY_HIP(hipMemcpy(L.rot_freq, freq.data(), std::max<size_t>(1, L.d.rot_dims / 2) * sizeof(float), hipMemcpyHostToDevice));
            if (L.d.mixer == ZG_LM_MIX_PARALLEL) {  // the values turn at the unscaled frequencies of their own size
                const int vd = L.d.vdim;
                std::vector<float> vf(std::max(1, vd / 2));
                for (int i = 0; i < vd / 2; ++i) vf[i] = (float)pow((double)L.d.rot_base, -2.0 * i / vd);
                ZG_LM_TRY_HIP(hipMemcpy(L.vfreq, vf.data(), vf.size() * sizeof(float), hipMemcpyHostToDevice));
            }
        }
    ZG_LM_TRY_HIP(hipStreamSynchronize(g->stream));
#undef ZG_LM_TRY_HIP
    g->slots.assign(g->NS, Slot());
    for (int p = g->n_pages - 1; p >= 0; --p) g->free_pages.push_back(p);
    *out = g;
    return ZG_OK;
}

int zg_lm_destroy(zg_lm* g) {
    if (!g) return ZG_OK;
    (void)hipSetDevice(g->device);
    if (g->stream) (void)hipStreamSynchronize(g->stream);
    for (auto& by_rows : g->decode_graph)
        for (hipGraphExec_t e : by_rows)
            if (e) (void)hipGraphExecDestroy(e);
    if (g->ev0) (void)hipEventDestroy(g->ev0);
    if (g->ev1) (void)hipEventDestroy(g->ev1);
    if (g->stream) (void)hipStreamDestroy(g->stream);
    if (g->h_meta) (void)hipHostFree(g->h_meta);
    if (g->h_logits) (void)hipHostFree(g->h_logits);
    if (g->h_small) (void)hipHostFree(g->h_small);
    if (g->h_u) (void)hipHostFree(g->h_u);
    if (g->arena) (void)hipFree(g->arena);
    delete g;
    return ZG_OK;
}

int zg_lm_load_tensor(zg_lm* g, const char* name, const float* data, size_t len) {
    ZG_REQUIRE(g && name && data, ZG_ERR_ARG, "lm_load_tensor: bad argument");
    ZG_HIP(hipSetDevice(g->device));
    auto it = g->tensors.find(name);
    ZG_REQUIRE(it != g->tensors.end(), ZG_ERR_ARG, "lm_load_tensor: the configuration has no tensor '%s'", name);
    Tensor& t = it->second;
    ZG_REQUIRE(len == t.rows * t.cols, ZG_ERR_SHAPE, "lm_load_tensor: '%s' has %zu elements, the configuration needs [%zu, %zu]", name, len, t.rows,
               t.cols);
    ZG_HIP(hipStreamSynchronize(g->stream));
    if (!t.matrix) {
        ZG_HIP(hipMemcpy(t.dev, data, len * sizeof(float), hipMemcpyHostToDevice));
    } else {
        std::vector<bf16_t> tmp(len);
        auto rne = [](float x) {
            uint32_t b;
            memcpy(&b, &x, 4);
            if ((b & 0x7F800000u) == 0x7F800000u) return (bf16_t)(b >> 16);  // inf / NaN keep their class
            b += 0x7FFFu + ((b >> 16) & 1u);
            return (bf16_t)(b >> 16);
        };
        if (t.transpose_heads > 0) {  // [heads * d][cols] -> [heads][cols][d]
            const size_t Hh = t.transpose_heads, dd = t.rows / Hh, cc = t.cols;
            for (size_t hh = 0; hh < Hh; ++hh)
                for (size_t i = 0; i < dd; ++i)
                    for (size_t c = 0; c < cc; ++c) tmp[(hh * cc + c) * dd + i] = rne(data[(hh * dd + i) * cc + c]);
        } else {
            for (size_t i = 0; i < len; ++i) tmp[i] = rne(data[i]);
        }
        if (t.ld > 0 && t.ld != t.cols)
            ZG_HIP(hipMemcpy2D(t.dev, t.ld * sizeof(bf16_t), tmp.data(), t.cols * sizeof(bf16_t), t.cols * sizeof(bf16_t), t.rows, hipMemcpyHostToDevice));
        else ZG_HIP(hipMemcpy(t.dev, tmp.data(), len * sizeof(bf16_t), hipMemcpyHostToDevice));
    }
    t.loaded = true;
    return ZG_OK;
}

int zg_lm_missing_tensors(zg_lm* g, size_t* count, char* names_out, size_t names_cap) {
    ZG_REQUIRE(g && count, ZG_ERR_ARG, "lm_missing_tensors: bad argument");
    size_t n = 0, off = 0;
    if (names_out && names_cap) names_out[0] = 0;
    for (auto& kv : g->tensors)
        if (!kv.second.loaded) {
            ++n;
            if (names_out && off + kv.first.size() + 2 < names_cap) {
                off += (size_t)snprintf(names_out + off, names_cap - off, "%s%s", off ? " " : "", kv.first.c_str());
            }
        }
    *count = n;
    return ZG_OK;
}

int zg_lm_init_random(zg_lm* g, uint64_t seed, float std_) {
    ZG_REQUIRE(g && std_ > 0.0f, ZG_ERR_ARG, "lm_init_random: bad argument");
    ZG_HIP(hipSetDevice(g->device));
    uint64_t idx = 0;
    for (auto& kv : g->tensors) {
        Tensor& t = kv.second;
        const size_t n = t.rows * t.cols;
        fill_kernel<<<(unsigned)((n + 255) / 256), 256, 0, g->stream>>>(t.dev, n, seed * 0x9E3779B97F4A7C15ULL + (++idx) * 0xD1B54A32D192ED03ULL, t.init,
                                                                        std_, t.cols, t.ld > 0 ? t.ld : t.cols);
        ZG_HIP(hipGetLastError());
        t.loaded = true;
    }
    ZG_HIP(hipStreamSynchronize(g->stream));
    return ZG_OK;
}

int zg_lm_seq_open(zg_lm* g, int* seq_out) {
    ZG_REQUIRE(g && seq_out, ZG_ERR_ARG, "lm_seq_open: bad argument");
    ZG_HIP(hipSetDevice(g->device));
    int sidx = -1;
    for (int i = 0; i < g->NS && sidx < 0; ++i)
        if (!g->slots[i].open) sidx = i;
    ZG_REQUIRE(sidx >= 0, ZG_ERR_SHAPE, "lm_seq_open: all %d state slots are in use", g->NS);
    // a slot starts from zeros: no previous row for the token shift, an empty recurrent state
    const size_t nsh = (size_t)g->n_passes * g->W;
    zero_kernel<<<(unsigned)((nsh + 255) / 256), 256, 0, g->stream>>>(g->shift_state + (size_t)sidx * nsh, nsh);
    ZG_HIP(hipGetLastError());
    if (g->hgrn_floats) {
        zero_kernel<<<(unsigned)((g->hgrn_floats + 255) / 256), 256, 0, g->stream>>>(g->hgrn_state + (size_t)sidx * g->hgrn_floats, g->hgrn_floats);
        ZG_HIP(hipGetLastError());
    }
    if (g->seq_floats) {
        zero_kernel<<<(unsigned)((g->seq_floats + 255) / 256), 256, 0, g->stream>>>(g->seq_state + (size_t)sidx * g->seq_floats, g->seq_floats);
        ZG_HIP(hipGetLastError());
    }
    Slot& sl = g->slots[sidx];
    sl.open = true;
    sl.len = 0;
    sl.pages.clear();
    sl.ring.assign(g->max_pages, 0);
    sl.first_live = 0;
    *seq_out = sidx;
    return ZG_OK;
}

int zg_lm_seq_close(zg_lm* g, int seq) {
    ZG_REQUIRE(g && seq >= 0 && seq < g->NS && g->slots[seq].open, ZG_ERR_ARG, "lm_seq_close: sequence %d is not open", seq);
    Slot& sl = g->slots[seq];
    for (int p : sl.pages)
        if (p >= 0) g->free_pages.push_back(p);
    sl.pages.clear();
    sl.open = false;
    sl.len = 0;
    return ZG_OK;
}

int zg_lm_seq_len(zg_lm* g, int seq, size_t* len_out) {
    ZG_REQUIRE(g && len_out && seq >= 0 && seq < g->NS && g->slots[seq].open, ZG_ERR_ARG, "lm_seq_len: sequence %d is not open", seq);
    *len_out = g->slots[seq].len;
    return ZG_OK;
}

int zg_lm_free_tokens(zg_lm* g, size_t* tokens_out) {
    ZG_REQUIRE(g && tokens_out, ZG_ERR_ARG, "lm_free_tokens: bad argument");
    *tokens_out = g->free_pages.size() * (size_t)g->P;
    return ZG_OK;
}

int zg_lm_step(zg_lm* g, const zg_lm_entry* entries, size_t n_entries, float* logits_out, size_t logits_len) {
    if (g) {
        size_t missing = 0;
        zg_lm_missing_tensors(g, &missing, nullptr, 0);
        ZG_REQUIRE(missing == 0, ZG_ERR_NOT_INITIALIZED, "lm_step: %zu tensors of the configuration have not been loaded", missing);
    }
    return step_impl(g, entries, n_entries, logits_out, logits_len, nullptr);
}

int zg_lm_generate(zg_lm* g, const int32_t* prompts, size_t prompt_stride, const size_t* prompt_lens, size_t n_prompts, size_t n_new, float temp,
                   uint64_t seed, int32_t* out_tokens, size_t out_len) {
    ZG_REQUIRE(g && prompts && prompt_lens && out_tokens && n_prompts >= 1 && temp >= 0.0f, ZG_ERR_ARG, "lm_generate: bad argument");
    ZG_REQUIRE(out_len >= n_prompts * n_new, ZG_ERR_SHAPE, "lm_generate: out_tokens needs %zu elements", n_prompts * n_new);
    ZG_REQUIRE(n_prompts <= (size_t)g->logit_rows, ZG_ERR_UNSUPPORTED, "lm_generate: %zu prompts (at most %d at a time)", n_prompts, g->logit_rows);
    size_t missing = 0;
    zg_lm_missing_tensors(g, &missing, nullptr, 0);
    ZG_REQUIRE(missing == 0, ZG_ERR_NOT_INITIALIZED, "lm_generate: %zu tensors of the configuration have not been loaded", missing);
    for (size_t b = 0; b < n_prompts; ++b)
        ZG_REQUIRE(prompt_lens[b] >= 1 && prompt_lens[b] <= prompt_stride, ZG_ERR_ARG, "lm_generate: prompt %zu has %zu tokens", b, prompt_lens[b]);
    if (n_new == 0) return ZG_OK;
    std::vector<int> seqs;
    int status = ZG_OK;
    for (size_t b = 0; b < n_prompts && status == ZG_OK; ++b) {
        int sq = -1;
        status = zg_lm_seq_open(g, &sq);
        if (status == ZG_OK) seqs.push_back(sq);
    }
    std::vector<int32_t> cur(n_prompts), zero(n_prompts, 0), last(n_prompts);
    const Sampler sm{temp, seed, cur.data()};
    std::vector<zg_lm_entry> ent(n_prompts);
    float decode_ms = 0.0f;
    size_t decode_steps = 0;
    for (size_t i = 0; i < n_new && status == ZG_OK; ++i) {
        for (size_t b = 0; b < n_prompts; ++b) {
            ent[b].seq = seqs[b];
            if (i == 0) {  // the prompts, cut into portions by the step
                ent[b].tokens = prompts + b * prompt_stride;
                ent[b].n_tokens = prompt_lens[b];
                last[b] = (int32_t)(prompt_lens[b] - 1);
                ent[b].want = &last[b];
            } else {
                ent[b].tokens = &out_tokens[b * n_new + i - 1];
                ent[b].n_tokens = 1;
                ent[b].want = &zero[b];
            }
            ent[b].n_want = 1;
        }
        status = step_impl(g, ent.data(), n_prompts, nullptr, 0, &sm);
        if (status != ZG_OK) break;
        if (i > 0) {
            decode_ms += g->last_step_ms;
            ++decode_steps;
        }
        for (size_t b = 0; b < n_prompts; ++b) out_tokens[b * n_new + i] = cur[b];
    }
    g->last_decode_ms = decode_steps ? decode_ms / (float)decode_steps : 0.0f;
    for (int sq : seqs) zg_lm_seq_close(g, sq);
    return status;
}

int zg_lm_set_trace(zg_lm* g, float* trace_out, size_t trace_floats) {
    ZG_REQUIRE(g, ZG_ERR_ARG, "lm_set_trace: bad argument");
    g->trace = trace_out;
    g->trace_floats = trace_out ? trace_floats : 0;
    return ZG_OK;
}

int zg_lm_last_ms(zg_lm* g, float* step_ms, float* decode_ms_per_step) {
    ZG_REQUIRE(g, ZG_ERR_ARG, "lm_last_ms: bad argument");
    if (step_ms) *step_ms = g->last_step_ms;
    if (decode_ms_per_step) *decode_ms_per_step = g->last_decode_ms;
    return ZG_OK;
}

}  // extern "C"
