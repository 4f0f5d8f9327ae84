// gl3_hybrid.h — plan state of the layer-list family (GL3_ARCH_LAYERLIST) and the entry points the C-ABI dispatches to.
#pragma once
#include <string>
#include <vector>

#include "gl3_ctx.h"

constexpr int HY_KSPLIT = 4;     // most partial sums a K-split output / down projection leaves for the streams kernel to add
constexpr int HY_YPARTS = 2 * HY_KSPLIT;      // copies of y: in a parallel block the mixer's and the feed-forward's parts lie side by side

struct HyMat {                 // [rows][ld] of the plan's matrix type (bfloat16 or float32), K-contiguous, zero padded
    void* w = nullptr;
    int rows = 0, k = 0, ld = 0;
};

struct HyLayer {
    gl3_layer_desc d{};
    // fused input projection of the mixer: attention q | k | v | gate; latent q | latent | gate; ssm z | x | B | C | dt; matrix memory
    // q | k | v | gate | input gate | forget gate.  A layer with two mixers side by side keeps the second one in `side`: its rows follow
    // the first mixer's in the layer's proj, its output columns follow the first mixer's in mixo and in o (the offsets below count from
    // the start of the fused row; proj, o and pbias of `side` are unused / borrowed)
    HyMat proj;
    int q_off = 0, k_off = 0, v_off = 0, g_off = 0, c_off = 0, i_off = 0, f_off = 0;
    int o0 = 0;                // first column of this mixer's heads in mixo and o
    int mo_total = 0;          // columns of o: this mixer's heads * vdim plus the side mixer's
    float out_mul = 1.f;
    HyLayer* side = nullptr;   // owned
    HyMat o;                   // the mixer's output projection [width x mo_total]
    float* pbias = nullptr;    // bias per row of the fused projection (null: no mixer of the layer has biases)
    float *qn = nullptr, *kn = nullptr, *sink = nullptr;      // attention: weights of the whole-projection q / k norms, learned sink logits
    float* decay = nullptr;    // matrix memory: fixed decay per head
    size_t off_pk = 0, off_pv = 0, off_m = 0;                 // float offsets inside a slot: pooled key / value rows, running maxima of the gates
    HyMat gu, down;            // feed-forward (in a mixture of experts: the shared expert): gate / up rows in blocks of 32 + 32 (2 ff_pad rows), down [width x ff_pad]
    int ff_pad = 0;
    int dense_ff = 0;          // width of that feed-forward (d.ff, or d.shared_ff in a mixture of experts; 0 = none)
    float dense_limit = 0.f;
    // mixture of experts: router rows (+ one row: the shared expert's gate); the routed experts stacked, each laid out like gu / down
    HyMat router, egu, edown;
    int eff_pad = 0;
    // plain-residual designs: weights of the depth average [layer + 2]; per-layer token input
    float* depth_mix = nullptr;
    HyMat side_gate, side_proj;
    float* side_norm = nullptr;
    float *rot_freq = nullptr, *vrot_freq = nullptr;       // rotary tables: [rot_dims / 2] (position scaling applied), [vdim / 2]
    float *norm1 = nullptr, *norm2 = nullptr;
    float* hc[2][3] = {};      // per sublayer: in [S], out [S], mix [S x S]
    // latent: norm weight; key expansion [H D][R] (as stored: rows for the expansion GEMM, and [h][d][r] for carrying a query into the latent's
    // space); value expansion as stored [H V][R] (GEMM) and transposed [H][R][V] (expansion of a weighted sum of latents)
    // With a rotated part (rot_dim > 0) the cached row is [latent | turned key part] (Re = kv_rank + rot_dim entries) and a query head has
    // De = dim + rot_dim entries; the expansions are padded to these sizes (key expansion: identity behind the latent's columns, value
    // expansion: zeros), so every kernel of the latent path runs on (De, Re) as it does on (dim, kv_rank) without a rotated part.
    float *lat_norm = nullptr, *wk = nullptr, *wv = nullptr, *wvT = nullptr;
    int De = 0, Re = 0;
    HyMat uq;                  // latent with q_rank: query expansion [heads De x q_rank]
    float* qlat_norm = nullptr;// norm weight of the query latent [q_rank]
    double* lat_freq = nullptr;// latent with a rotated part: frequencies [rot_dim / 2] in double
    float rot_mscale = 1.f;    // multiplier of cos and sin of that part
    float *norm1b = nullptr, *norm2b = nullptr;      // post norms of the two sublayers
    float* route_bias = nullptr;                     // mixture of experts: added to the scores for the choice
    float *conv_w = nullptr, *conv_b = nullptr, *dt_bias = nullptr, *a_log = nullptr, *dskip = nullptr, *ssm_norm = nullptr;
    size_t off_k = 0, off_v = 0, off_state = 0, off_tail = 0;       // float offsets inside a sequence slot
    uint64_t have = 0;
};

struct gl3_hybrid_state {
    bool f32 = false;          // GL3_FLAG_F32_COMPUTE
    int S = 1, W = 0, mb = 1, n_seqs = 1, want_cap = 1;
    bool plain = false;        // one residual stream without stream tables (gl3_model_desc.streams == 0)
    bool parallel = false;     // plain: one norm per layer, mixer and feed-forward read it and are added together (gl3_model_desc.parallel_block)
    float resid_mul = 1.f, logit_mul = 1.f;
    float emb_scale = 1.f, norm_offset = 0.f;
    int side_dim = 0, side_ld = 0, max_top = 0;
    bool depth = false;
    bool post_norms = false;   // every sublayer's output passes an RMS norm with its own weight before it joins the residual
    float softcap = 0.f;       // logits <- cap tanh(logits / cap); 0 = none
    void* cq = nullptr;        // latent with q_rank: the normed query latents [mb][max q_rank], matrix type
    float* qfull = nullptr;    // ... and the expanded queries [mb][max heads De]
    HyMat side_emb;            // [vocab][layers * side_dim]
    // [layers + 1][mb][W]; K-split parts of [mb][side_dim] and of [mb][experts + 1]; the shared expert's gate logit [mb]; [mb top]; [mb top][W]
    float *hist = nullptr, *side_z = nullptr, *moe_z = nullptr, *sgz = nullptr, *wsel = nullptr, *eout = nullptr;
    void *xb = nullptr, *side_g = nullptr, *ea = nullptr, *eact = nullptr;                              // matrix type: [mb][W]; [mb][side_ld]; [mb top][W]; [mb top][eff_pad]
    int *sel = nullptr, *pair_row = nullptr, *tiles = nullptr, *ntiles = nullptr;
    std::vector<HyLayer> L;
    HyMat emb, head;
    float* final_norm = nullptr;
    uint64_t have = 0;
    // sequence slots: cache rows and recurrent state of every layer, [n_seqs][slot_floats]
    float* slots = nullptr;
    size_t slot_floats = 0;
    std::vector<char> busy;
    std::vector<int> len;      // tokens a slot holds
    // scratch of one portion of a step (<= mb tokens)
    float *X = nullptr, *proj = nullptr, *y = nullptr, *conv = nullptr, *ssm_y = nullptr, *qa = nullptr, *oc = nullptr, *kx = nullptr, *vx = nullptr, *part_acc = nullptr, *part_ml = nullptr;
    float *gates = nullptr, *rowr = nullptr;     // matrix memory: a, b, e^(-m) per (token, head), [3][mb][max heads]; attention: 1 / rms of the whole q and k rows [mb][2]
    int max_heads = 1;
    void *h = nullptr, *mixo = nullptr, *xw = nullptr;
    float *logits = nullptr, *taps = nullptr, *ones = nullptr;
    int *tokens = nullptr, *dyn = nullptr, *want = nullptr;
    int *h_tokens = nullptr, *h_dyn = nullptr, *h_want = nullptr;    // pinned
    float* h_logits = nullptr;                                       // pinned [want_cap][vocab]
    size_t part_rows = 0;
    int last_n = 0;
    int y_parts = 1;           // partial sums the last output / down projection left in y (added by the streams kernel)
};

int32_t gl3_hy_create(const gl3_model_desc* desc, gl3_ctx** out, std::string& err);
void gl3_hy_destroy(gl3_ctx* ctx);                 // frees ctx->hy only
int32_t gl3_hy_upload(gl3_ctx* ctx, int32_t id, int32_t layer, const void* host, uint64_t bytes, int32_t type);
int32_t gl3_hy_finalize(gl3_ctx* ctx);
int32_t gl3_hy_step(gl3_ctx* ctx, int32_t seq, const int32_t* tokens, int32_t n, int32_t start_pos, const int32_t* want, int32_t n_want,
                    float* logits_out);
int32_t gl3_hy_argmax(gl3_ctx* ctx, int32_t* out);                  // greedy id of the last step's first wanted row
int32_t gl3_hy_seq_acquire(gl3_ctx* ctx, int32_t* seq_out);
int32_t gl3_hy_seq_release(gl3_ctx* ctx, int32_t seq);
int32_t gl3_hy_layer_rows(gl3_ctx* ctx, int32_t layer, float* out, int32_t n);
int32_t gl3_hy_reset(gl3_ctx* ctx);
// one GEMM class of the family timed alone (bench.py): rows x k matrix, m tokens, mean microseconds per launch
int32_t gl3_hy_profile_gemm(int32_t device, int32_t f32, int32_t rows, int32_t k, int32_t m, int32_t glu, int32_t iters, double* out_us);
