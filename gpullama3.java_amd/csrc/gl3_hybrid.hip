// gl3_hybrid.hip — the layer-list family (GL3_ARCH_LAYERLIST) behind the C-ABI: a model is a list of layers, each with its own token mixer
// (softmax attention over cached keys / values, attention over a cached low-rank latent — optionally with a query latent, a rotated key
// part shared by all heads and rows that a later layer reads too —, a state-space recurrence, a matrix memory with a fixed decay or
// exponential gates), an optional feed-forward (gated or relu^2, dense or a mixture of experts with a shared expert and a sigmoid or
// softmax router), and either several residual streams that per-sublayer tables read from and write to, or one plain residual stream
// with an optional per-layer token input, a weighted average over all earlier layers' results, one norm for both sublayers of a layer, or
// a norm behind every sublayer as well as in front of it.
//
// Plan: matrices live in HBM as bfloat16 (default) or widened to float32 (GL3_FLAG_F32_COMPUTE); every sequence slot owns the cache
// rows and the recurrent state of all layers; a step runs the next n tokens of one slot in portions of at most max_batch tokens:
//   streams kernel (tables + norm) -> input GEMM of the mixer -> mixer kernels -> output GEMM -> streams kernel (write-back of this
//   sublayer fused with the read + norm of the next) -> gate/up GEMM with the activation in its epilogue -> down GEMM -> streams kernel
// and the logits of the wanted rows only.  Portions of <= 8 tokens (decode) take the matvec kernels instead of the MFMA tiles.
#include <algorithm>
#include <cmath>
#include <cstring>

#include "gl3_hybrid.h"
#include "gl3_decode_kernels.h"      // argmax_kernel
#include "gl3_hy_kernels.h"
#include "gl3_hy_plain_kernels.h"

using gl3::AMX_WGS;
using gl3::argmax_kernel;

#define HY_HIP(call)                                                                                   \
    do {                                                                                               \
        hipError_t e_ = (call);                                                                        \
        if (e_ != hipSuccess) {                                                                        \
            ctx->err = std::string(#call) + ": " + hipGetErrorString(e_);                              \
            return e_ == hipErrorOutOfMemory ? GL3_E_OOM : GL3_E_HIP;                                  \
        }                                                                                              \
    } while (0)

static inline int hy_cdiv(int a, int b) { return (a + b - 1) / b; }
constexpr int HY_MOE_BM = 64;        // rows per tile of the grouped expert GEMMs
constexpr int HY_LATENT_DIRECT = 512;   // longest cached latent row that decode steps score in the latent's space (value columns per lane of the attention core)
constexpr int HY_ZSPLIT = 16;        // most K-split parts of a product with very few result rows (router, token input's gate): its consumer kernel adds them
static inline float hy_bf16_to_f32(uint16_t v) { uint32_t u = (uint32_t)v << 16; float f; memcpy(&f, &u, 4); return f; }
static inline uint16_t hy_f32_to_bf16(float f) {
    uint32_t u; memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

template <typename P>
static int32_t hy_alloc(gl3_ctx* ctx, P** p, size_t bytes) {
    HY_HIP(hipMalloc((void**)p, bytes + GL3_TAIL_PAD));
    HY_HIP(hipMemset(*p, 0, bytes + GL3_TAIL_PAD));
    return GL3_OK;
}
static int32_t hy_alloc_mat(gl3_ctx* ctx, HyMat& m, int rows, int k, int ld) {
    m.rows = rows; m.k = k; m.ld = ld;
    return hy_alloc(ctx, &m.w, (size_t)rows * ld * (ctx->hy->f32 ? 4 : 2));
}

// ---- shapes -----------------------------------------------------------------------------------------------------------------------
static int hy_gate_rows(const gl3_layer_desc& d) { return d.mixer == GL3_MIX_MEMORY ? d.heads * d.vdim : d.out_gate == 2 ? d.heads : d.out_gate ? d.heads * d.vdim : 0; }
// rows of ONE mixer's part of the fused input projection
static int hy_proj_rows(const gl3_layer_desc& d) {
    switch (d.mixer) {
        case GL3_MIX_ATTENTION: return d.heads * d.dim + d.kv_heads * d.dim + d.kv_heads * d.vdim + hy_gate_rows(d);
        case GL3_MIX_LATENT: return (d.q_rank > 0 ? d.q_rank : d.heads * (d.dim + d.rot_dim)) + (d.kv_share > 0 ? 0 : d.kv_rank + d.rot_dim) + hy_gate_rows(d);
        case GL3_MIX_MEMORY: return 2 * d.heads * d.dim + 2 * d.heads * d.vdim + (d.mem_gates == GL3_MEM_EXP_GATES ? 2 * d.heads : 0);
        default: return 2 * d.heads * d.vdim + 2 * d.groups * d.state + d.heads;
    }
}
static int hy_mix_out(const gl3_layer_desc& d) { return d.heads * d.vdim; }
// the fused input projection may come in K-split parts (room for HY_KSPLIT copies in the plan's scratch)
static bool hy_narrow_proj(const gl3_layer_desc& d) { return d.mixer == GL3_MIX_LATENT && d.q_rank > 0; }
static bool hy_has_bias(const gl3_layer_desc& d) { return (d.mixer == GL3_MIX_ATTENTION && d.qk_bias) || (d.mixer == GL3_MIX_MEMORY && d.mem_gates == GL3_MEM_EXP_GATES); }
static int hy_conv_ch(const gl3_layer_desc& d) { return d.heads * d.vdim + 2 * d.groups * d.state; }

static const char* hy_check_layer(const gl3_layer_desc& d) {
    if (d.heads < 1 || d.vdim < 1) return "heads and vdim must be positive";
    if (d.ff < 0) return "ff must be >= 0";
    if (d.out_gate < 0 || d.out_gate > 2) return "out_gate must be 0, 1 or 2";
    if (d.experts < 0 || d.shared_ff < 0) return "experts and shared_ff must be >= 0";
    if (d.experts > 0) {
        if (d.ff < 1) return "mixture of experts: ff (one expert's width) must be positive";
        if (d.ff_act == 2) return "mixture of experts: the experts are gated (ff_act 0 or 1)";
        if (d.experts + (d.shared_ff > 0 ? 1 : 0) > 64 * HY_RT_PER) return "mixture of experts: at most 1024 router rows (experts, plus one for a shared expert's gate)";
        if (d.top < 1 || d.top > d.experts || d.top > 64) return "mixture of experts: 1 <= top <= min(experts, 64)";
    } else if (d.shared_ff > 0)
        return "a shared expert needs a mixture of experts";
    if (d.mixer != GL3_MIX_ATTENTION && (d.v_unit_norm || d.v_rot || d.window > 0 || d.keep_first > 0 || d.pool > 0 || d.qk_bias))
        return "value norm / rotation, windows, pooled blocks and q / k / v biases belong to the attention mixer";
    if (d.mixer != GL3_MIX_ATTENTION && d.mixer != GL3_MIX_MEMORY && d.rot_dims) return "rotary positions belong to the attention and matrix-memory mixers";
    if (d.ff_act < 0 || d.ff_act > 2) return "ff_act must be 0, 1 or 2";
    if (d.mixer != GL3_MIX_LATENT && (d.q_rank || d.rot_dim || d.kv_share)) return "q_rank, rot_dim and kv_share belong to the latent attention";
    if (d.mixer != GL3_MIX_MEMORY && (d.mem_qkv_act || d.mem_norm_whole)) return "mem_qkv_act and mem_norm_whole belong to the matrix memory";
    if (d.mixer == GL3_MIX_ATTENTION) {
        if (d.kv_heads < 1 || d.heads % d.kv_heads) return "attention: heads must be a multiple of kv_heads";
        if (d.dim < 1) return "attention: dim must be positive";
        if (d.vdim > 512 || d.dim > 1024) return "attention: dim <= 1024 and vdim <= 512";
        if (d.rot_dims < 0 || d.rot_dims > d.dim || (d.rot_dims & 1)) return "attention: rot_dims must be even and at most dim";
        if ((d.rot_dims || d.v_rot) && !(d.rot_base > 0.f)) return "attention: rot_base must be positive";
        if (d.v_rot && (d.vdim & 1)) return "attention: rotated values need an even vdim";
        if (d.keep_first < 0) return "attention: keep_first must be >= 0";
        if (d.qk_unit_norm < 0 || d.qk_unit_norm > 2 || d.softmax_sink < 0 || d.softmax_sink > 2) return "attention: qk_unit_norm and softmax_sink must be 0, 1 or 2";
        if (d.pool < 0 || (d.pool > 0 && d.window <= 0)) return "attention: pooled blocks need a window";
        if (d.pool > 0 && d.slope_log2 != 0.f) return "attention: pooled blocks have no distance term";
    } else if (d.mixer == GL3_MIX_LATENT) {
        if (d.dim < 1 || d.kv_rank < 1) return "latent attention: dim and kv_rank must be positive";
        if (d.rot_dim < 0 || (d.rot_dim & 1)) return "latent attention: rot_dim must be even and >= 0";
        if (d.kv_rank + d.rot_dim > 8192 || d.dim + d.rot_dim > 1024 || d.vdim > 512) return "latent attention: kv_rank + rot_dim <= 8192, dim + rot_dim <= 1024, vdim <= 512";
        if (d.rot_dim > 0 && !(d.rot_base > 0.f)) return "latent attention: rot_base must be positive";
        if (d.rot_dim > 0 && d.rot_yarn_factor > 0.f && !(d.rot_yarn_original > 0.f && d.rot_yarn_fast > 0.f && d.rot_yarn_slow > 0.f && d.rot_base != 1.f))
            return "latent attention: scaled frequencies need original, fast and slow > 0";
        if (d.q_rank < 0 || d.kv_share < 0) return "latent attention: q_rank and kv_share must be >= 0";
    } else if (d.mixer == GL3_MIX_MEMORY) {
        if (d.dim < 1 || d.dim > 2048) return "matrix memory: 1 <= dim <= 2048";
        if (d.rot_dims < 0 || d.rot_dims > d.dim || (d.rot_dims & 1)) return "matrix memory: rot_dims must be even and at most dim";
        if (d.rot_dims && !(d.rot_base > 0.f)) return "matrix memory: rot_base must be positive";
        if (d.mem_gates != GL3_MEM_DECAY && d.mem_gates != GL3_MEM_EXP_GATES) return "matrix memory: unknown mem_gates";
        if (d.mem_gates == GL3_MEM_DECAY && !d.mem_decay) return "matrix memory: a fixed decay needs mem_decay";
        if (d.mem_gates == GL3_MEM_EXP_GATES && !(d.mem_gate_cap > 0.f)) return "matrix memory: mem_gate_cap must be positive";
    } else if (d.mixer == GL3_MIX_SSM) {
        if (d.state < 1 || d.state > 2048) return "ssm: 1 <= state <= 2048";
        if (d.groups < 1 || d.heads % d.groups) return "ssm: heads must be a multiple of groups";
        if (d.norm_groups < 1 || (d.heads * d.vdim) % d.norm_groups) return "ssm: heads * vdim must be a multiple of norm_groups";
        if (d.conv < 1 || d.conv > 64) return "ssm: 1 <= conv <= 64";
    } else
        return "unknown mixer";
    return nullptr;
}

int32_t gl3_hy_create(const gl3_model_desc* desc, gl3_ctx** out, std::string& err) {
    if (desc->n_layers < 1 || !desc->layer_descs) { err = "layer-list family: n_layers >= 1 and layer_descs are required"; return GL3_E_ARG; }
    if (desc->streams < 0 || desc->streams > HY_MAX_STREAMS) { err = "layer-list family: 0 <= streams <= 8"; return GL3_E_ARG; }
    if (desc->streams > 0 && (desc->side_dim || desc->depth_mix)) { err = "layer-list family: the per-layer token input and the depth average need the plain residual (streams = 0)"; return GL3_E_ARG; }
    if (desc->side_dim < 0) { err = "layer-list family: side_dim must be >= 0"; return GL3_E_ARG; }
    for (int l = 0; l < desc->n_layers && desc->streams > 0; ++l)
        if (desc->layer_descs[l].experts > 0) { err = "layer-list family: a mixture of experts needs the plain residual (streams = 0)"; return GL3_E_ARG; }
    if (desc->dim < 1 || desc->vocab < 1 || desc->ctx < 1) { err = "layer-list family: dim, vocab and ctx must be positive"; return GL3_E_ARG; }
    if (desc->weight_type != GL3_TYPE_BF16 && desc->weight_type != GL3_TYPE_F32) { err = "layer-list family: weight_type must be GL3_TYPE_BF16 (or GL3_TYPE_F32)"; return GL3_E_UNSUPPORTED; }
    if (desc->tp_size > 1) { err = "layer-list family: tensor parallelism is not built"; return GL3_E_UNSUPPORTED; }
    if (desc->post_norms && (desc->streams > 0 || desc->side_dim || desc->depth_mix || desc->parallel_block)) { err = "layer-list family: post norms need the plain residual without token input, depth average and parallel block"; return GL3_E_ARG; }
    if (desc->logit_softcap < 0.f) { err = "layer-list family: logit_softcap must be >= 0"; return GL3_E_ARG; }
    if (desc->parallel_block && (desc->streams > 0 || desc->side_dim || desc->depth_mix)) { err = "layer-list family: the parallel block needs the plain residual without token input and depth average"; return GL3_E_ARG; }
    for (int l = 0; l < desc->n_layers; ++l) {
        const gl3_layer_desc& ld = desc->layer_descs[l];
        if (const char* m = hy_check_layer(ld)) { err = "layer " + std::to_string(l) + ": " + m; return GL3_E_ARG; }
        if (desc->parallel_block && ld.experts > 0) { err = "layer-list family: the parallel block has a dense feed-forward"; return GL3_E_ARG; }
        if (ld.mixer == GL3_MIX_LATENT && ld.kv_share > 0) {          // the cache it reads: an earlier latent layer with rows of its own and the same row layout
            const int j = ld.kv_share - 1;
            const gl3_layer_desc* o = j < l ? &desc->layer_descs[j] : nullptr;
            if (!o || o->mixer != GL3_MIX_LATENT || o->kv_share > 0 || o->kv_rank != ld.kv_rank || o->rot_dim != ld.rot_dim) {
                err = "layer " + std::to_string(l) + ": kv_share must name an earlier latent-attention layer with a cache of its own and the same kv_rank and rot_dim"; return GL3_E_ARG;
            }
        }
        if (ld.beside) {
            if (ld.beside->mixer == GL3_MIX_LATENT || ld.mixer == GL3_MIX_LATENT || ld.beside->mixer == GL3_MIX_SSM || ld.mixer == GL3_MIX_SSM) {
                err = "layer " + std::to_string(l) + ": only attention and matrix-memory mixers can stand side by side"; return GL3_E_ARG;
            }
            if (const char* m = hy_check_layer(*ld.beside)) { err = "layer " + std::to_string(l) + ", second mixer: " + m; return GL3_E_ARG; }
        }
    }
    gl3_ctx* ctx = new gl3_ctx();
    ctx->d = *desc;
    ctx->d.layer_descs = nullptr;
    ctx->n_seqs = desc->n_seqs < 1 ? 1 : desc->n_seqs;
    gl3_hybrid_state* h = ctx->hy = new gl3_hybrid_state();
    h->f32 = (desc->flags & GL3_FLAG_F32_COMPUTE) != 0;
    h->plain = desc->streams == 0;
    h->parallel = desc->parallel_block != 0;
    h->resid_mul = (h->parallel && desc->residual_scale != 0.f) ? desc->residual_scale : 1.f;
    h->logit_mul = desc->logit_scale != 0.f ? desc->logit_scale : 1.f;
    h->emb_scale = desc->embedding_scale != 0.f ? desc->embedding_scale : 1.f;
    h->norm_offset = desc->norm_offset;
    h->side_dim = desc->side_dim; h->side_ld = hy_cdiv(std::max(1, desc->side_dim), 8) * 8;
    h->depth = desc->depth_mix != 0;
    h->post_norms = desc->post_norms != 0;
    h->softcap = desc->logit_softcap;
    h->S = std::max(1, desc->streams); h->W = desc->dim; h->mb = std::max(1, desc->max_batch); h->n_seqs = ctx->n_seqs;
    h->want_cap = std::min(h->mb, 256);
    h->busy.assign(h->n_seqs, 0); h->len.assign(h->n_seqs, 0);
    auto fail = [&](int32_t code) { err = ctx->err; gl3_hy_destroy(ctx); if (ctx->stream) hipStreamDestroy(ctx->stream); if (ctx->argmax) hipFree(ctx->argmax);
                                    if (ctx->h_argmax) hipHostFree(ctx->h_argmax); if (ctx->h_dyn) hipHostFree(ctx->h_dyn); delete ctx; return code; };
#define TRY(x) do { int32_t r_ = (x); if (r_ != GL3_OK) return fail(r_); } while (0)
#define TRYHIP(call) do { hipError_t e_ = (call); if (e_ != hipSuccess) { ctx->err = std::string(#call) + ": " + hipGetErrorString(e_); return fail(e_ == hipErrorOutOfMemory ? GL3_E_OOM : GL3_E_HIP); } } while (0)
    TRYHIP(hipSetDevice(desc->device));
    TRYHIP(hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking));
    const int W = h->W, S = h->S, mb = h->mb, V = desc->vocab, C = desc->ctx;
    const size_t es = h->f32 ? 4 : 2;
    TRY(hy_alloc_mat(ctx, h->emb, V, W, W));
    TRY(hy_alloc_mat(ctx, h->head, V, W, W));
    TRY(hy_alloc(ctx, &h->final_norm, (size_t)W * 4));
    h->L.resize(desc->n_layers);
    size_t slot = 0;
    int max_proj = 1, max_mix = W, max_ch = 1, max_inner = 1, max_hr = 1, max_hdv = 1, max_kx = 0, max_vx = 0, max_rz = 0, max_top = 0, max_eff = 0, max_e = 0;
    if (h->side_dim > 0) TRY(hy_alloc_mat(ctx, h->side_emb, V, desc->n_layers * h->side_dim, desc->n_layers * h->side_dim));
    int max_heads = 1, max_qr = 0, max_qfull = 0;
    bool long_latent = false;
    // one mixer's share of the layer: its offsets in the fused projection row (p0 = its first row) and in mixo / o (o0 = its first
    // column), its vectors and tables, its part of the sequence slot
    auto setup_mixer = [&](HyLayer& Ly, int p0, int o0) -> int32_t {
        const gl3_layer_desc& d = Ly.d;
        Ly.o0 = o0;
        Ly.out_mul = d.out_scale != 0.f ? d.out_scale : 1.f;
        max_heads = std::max(max_heads, d.heads);
#define TRYM(x) do { int32_t r_ = (x); if (r_ != GL3_OK) return r_; } while (0)
        // rotary tables, made in double: entry i turns by pos * base^(-2 i / dims) (q / k: divided by the position scaling)
        auto table = [&](float** dst, int dims, double divide) -> int32_t {
            std::vector<float> f(dims / 2);
            for (int i = 0; i < dims / 2; ++i) f[i] = (float)(std::pow((double)d.rot_base, -2.0 * i / dims) / divide);
            int32_t r_ = hy_alloc(ctx, dst, f.size() * 4);
            if (r_ != GL3_OK) return r_;
            return hipMemcpy(*dst, f.data(), f.size() * 4, hipMemcpyHostToDevice) == hipSuccess ? GL3_OK : GL3_E_HIP;
        };
        if (d.mixer == GL3_MIX_ATTENTION) {
            Ly.q_off = p0; Ly.k_off = Ly.q_off + d.heads * d.dim; Ly.v_off = Ly.k_off + d.kv_heads * d.dim; Ly.g_off = Ly.v_off + d.kv_heads * d.vdim;
            if (d.rot_dims > 0) TRYM(table(&Ly.rot_freq, d.rot_dims, d.rot_divide > 0.f ? (double)d.rot_divide : 1.0));
            if (d.v_rot) TRYM(table(&Ly.vrot_freq, d.vdim, 1.0));
            Ly.off_k = slot; slot += (size_t)C * d.kv_heads * d.dim;
            Ly.off_v = slot; slot += (size_t)C * d.kv_heads * d.vdim;
            if (d.pool > 0) {          // one pooled row per complete block of `pool` positions
                Ly.off_pk = slot; slot += (size_t)(C / d.pool + 1) * d.kv_heads * d.dim;
                Ly.off_pv = slot; slot += (size_t)(C / d.pool + 1) * d.kv_heads * d.vdim;
            }
            if (d.qk_unit_norm == 2) {
                TRYM(hy_alloc(ctx, &Ly.qn, (size_t)d.heads * d.dim * 4));
                TRYM(hy_alloc(ctx, &Ly.kn, (size_t)d.kv_heads * d.dim * 4));
            }
            if (d.softmax_sink == 2) TRYM(hy_alloc(ctx, &Ly.sink, (size_t)d.heads * 4));
            max_hdv = std::max(max_hdv, d.heads * d.vdim);
        } else if (d.mixer == GL3_MIX_LATENT) {
            const int De = Ly.De = d.dim + d.rot_dim, Re = Ly.Re = d.kv_rank + d.rot_dim;
            Ly.q_off = p0; Ly.c_off = Ly.q_off + (d.q_rank > 0 ? d.q_rank : d.heads * De); Ly.g_off = Ly.c_off + (d.kv_share > 0 ? 0 : Re);
            if (d.kv_share > 0) Ly.off_k = Ly.off_v = h->L[d.kv_share - 1].off_k;          // another layer's rows
            else {
                Ly.off_k = Ly.off_v = slot; slot += (size_t)C * Re;
                TRYM(hy_alloc(ctx, &Ly.lat_norm, (size_t)d.kv_rank * 4));
            }
            TRYM(hy_alloc(ctx, &Ly.wk, (size_t)d.heads * De * Re * 4));
            TRYM(hy_alloc(ctx, &Ly.wv, (size_t)d.heads * d.vdim * Re * 4));
            TRYM(hy_alloc(ctx, &Ly.wvT, (size_t)d.heads * d.vdim * Re * 4));
            if (d.q_rank > 0) {
                TRYM(hy_alloc_mat(ctx, Ly.uq, d.heads * De, d.q_rank, d.q_rank));
                TRYM(hy_alloc(ctx, &Ly.qlat_norm, (size_t)d.q_rank * 4));
                max_qr = std::max(max_qr, d.q_rank); max_qfull = std::max(max_qfull, d.heads * De);
            }
            if (d.rot_dim > 0) {
                // frequencies of the rotated part, made in double: base^(-2 i / n), blended with the / factor frequency along a ramp over the
                // pair index when rot_yarn_factor > 0; cos and sin then carry the multiplier 0.1 ln(factor) + 1
                const int n = d.rot_dim;
                std::vector<double> f(n / 2);
                const double base = d.rot_base, factor = d.rot_yarn_factor;
                double lo = 0, hi = 0;
                if (factor > 0.0) {
                    auto where = [&](double turns) { return n * std::log((double)d.rot_yarn_original / (2.0 * M_PI * turns)) / (2.0 * std::log(base)); };
                    lo = std::max(std::floor(where(d.rot_yarn_fast)), 0.0);
                    hi = std::min(std::ceil(where(d.rot_yarn_slow)), (double)(n - 1));
                    Ly.rot_mscale = (float)(0.1 * std::log(factor) + 1.0);
                }
                for (int i = 0; i < n / 2; ++i) {
                    const double fi = std::pow(base, -2.0 * i / n);
                    const double ramp = factor > 0.0 ? std::min(1.0, std::max(0.0, (i - lo) / std::max(hi - lo, 0.001))) : 0.0;
                    f[i] = factor > 0.0 ? fi / factor * ramp + fi * (1.0 - ramp) : fi;
                }
                TRYM(hy_alloc(ctx, &Ly.lat_freq, f.size() * 8));
                if (hipMemcpy(Ly.lat_freq, f.data(), f.size() * 8, hipMemcpyHostToDevice) != hipSuccess) { ctx->err = "copy of the rotary table failed"; return GL3_E_HIP; }
            }
            if (Re <= HY_LATENT_DIRECT) max_hr = std::max(max_hr, d.heads * Re);
            else long_latent = true;
            max_hdv = std::max(max_hdv, std::max(Re <= HY_LATENT_DIRECT ? d.heads * Re : 0, d.heads * d.vdim));
            max_kx = std::max(max_kx, d.heads * De); max_vx = std::max(max_vx, d.heads * d.vdim);
        } else if (d.mixer == GL3_MIX_MEMORY) {
            const bool eg = d.mem_gates == GL3_MEM_EXP_GATES;
            Ly.d.kv_heads = d.heads;
            Ly.q_off = p0; Ly.k_off = Ly.q_off + d.heads * d.dim; Ly.v_off = Ly.k_off + d.heads * d.dim; Ly.g_off = Ly.v_off + d.heads * d.vdim;
            Ly.i_off = Ly.g_off + d.heads * d.vdim; Ly.f_off = Ly.i_off + d.heads;
            if (d.rot_dims > 0) TRYM(table(&Ly.rot_freq, d.rot_dims, d.rot_divide > 0.f ? (double)d.rot_divide : 1.0));
            const int P = d.vdim + (eg ? 1 : 0);             // exponential gates: one more state column carries the normaliser
            Ly.off_state = slot; slot += (size_t)d.heads * d.dim * P;
            if (eg) { Ly.off_m = slot; slot += (size_t)d.heads; }
            else {
                TRYM(hy_alloc(ctx, &Ly.decay, (size_t)d.heads * 4));
                if (hipMemcpy(Ly.decay, d.mem_decay, (size_t)d.heads * 4, hipMemcpyHostToDevice) != hipSuccess) { ctx->err = "copy of mem_decay failed"; return GL3_E_HIP; }
            }
            if (d.mem_norm_weight) TRYM(hy_alloc(ctx, &Ly.ssm_norm, (size_t)d.heads * d.vdim * 4));
            max_inner = std::max(max_inner, d.heads * P);
        } else {
            const int ch = hy_conv_ch(d), inner = d.heads * d.vdim;
            Ly.off_state = slot; slot += (size_t)d.heads * d.state * d.vdim;
            Ly.off_tail = slot; slot += (size_t)std::max(1, d.conv - 1) * ch;
            TRYM(hy_alloc(ctx, &Ly.conv_w, (size_t)ch * d.conv * 4));
            TRYM(hy_alloc(ctx, &Ly.conv_b, (size_t)ch * 4));
            TRYM(hy_alloc(ctx, &Ly.dt_bias, (size_t)d.heads * 4));
            TRYM(hy_alloc(ctx, &Ly.a_log, (size_t)d.heads * 4));
            TRYM(hy_alloc(ctx, &Ly.dskip, (size_t)d.heads * 4));
            TRYM(hy_alloc(ctx, &Ly.ssm_norm, (size_t)inner * 4));
            max_ch = std::max(max_ch, ch); max_inner = std::max(max_inner, inner);
        }
#undef TRYM
        Ly.d.mem_decay = nullptr;          // the caller's array is not kept
        Ly.d.beside = nullptr;
        return GL3_OK;
    };
    for (int l = 0; l < desc->n_layers; ++l) {
        HyLayer& Ly = h->L[l];
        const gl3_layer_desc& d = Ly.d = desc->layer_descs[l];
        const gl3_layer_desc* bd = d.beside;
        if (bd) {
            Ly.side = new HyLayer();
            Ly.side->d = *bd;
            Ly.side->d.ff = 0; Ly.side->d.experts = 0; Ly.side->d.shared_ff = 0;
        }
        const int np1 = hy_proj_rows(d), mo1 = hy_mix_out(d);
        const int np = np1 + (bd ? hy_proj_rows(*bd) : 0), mo = mo1 + (bd ? hy_mix_out(*bd) : 0);
        const bool bias = hy_has_bias(d) || (bd && hy_has_bias(*bd));
        Ly.mo_total = mo;
        TRY(hy_alloc_mat(ctx, Ly.proj, np, W, W));
        TRY(hy_alloc_mat(ctx, Ly.o, W, mo, mo));
        if (bias) TRY(hy_alloc(ctx, &Ly.pbias, (size_t)np * 4));
        TRY(hy_alloc(ctx, &Ly.norm1, (size_t)W * 4));
        for (int q = 0; q < (d.ff > 0 ? 2 : 1) && !h->plain; ++q) {
            TRY(hy_alloc(ctx, &Ly.hc[q][0], (size_t)S * 4));
            TRY(hy_alloc(ctx, &Ly.hc[q][1], (size_t)S * 4));
            TRY(hy_alloc(ctx, &Ly.hc[q][2], (size_t)S * S * 4));
        }
        max_proj = std::max(max_proj, (hy_narrow_proj(d) && !bd ? HY_KSPLIT : 1) * np); max_mix = std::max(max_mix, mo);
        TRY(setup_mixer(Ly, 0, 0));
        if (Ly.side) {
            Ly.side->pbias = Ly.pbias; Ly.side->mo_total = mo;
            TRY(setup_mixer(*Ly.side, np1, mo1));
        }
        Ly.dense_ff = d.experts > 0 ? d.shared_ff : d.ff;
        Ly.dense_limit = d.experts > 0 ? d.shared_limit : d.ff_limit;
        if (d.ff > 0 && !h->parallel) TRY(hy_alloc(ctx, &Ly.norm2, (size_t)W * 4));
        if (h->post_norms) {
            TRY(hy_alloc(ctx, &Ly.norm1b, (size_t)W * 4));
            if (d.ff > 0) TRY(hy_alloc(ctx, &Ly.norm2b, (size_t)W * 4));
        }
        if (Ly.dense_ff > 0) {
            Ly.ff_pad = hy_cdiv(Ly.dense_ff, 32) * 32;
            TRY(hy_alloc_mat(ctx, Ly.gu, (d.experts == 0 && d.ff_act == 2 ? 1 : 2) * Ly.ff_pad, W, W));          // without a gate: the up rows alone
            TRY(hy_alloc_mat(ctx, Ly.down, W, Ly.ff_pad, Ly.ff_pad));
            max_mix = std::max(max_mix, Ly.ff_pad);
        }
        if (d.experts > 0) {
            Ly.eff_pad = hy_cdiv(d.ff, 32) * 32;
            TRY(hy_alloc_mat(ctx, Ly.router, d.experts + (d.shared_ff > 0 && !d.shared_ungated ? 1 : 0), W, W));
            if (d.route_bias) TRY(hy_alloc(ctx, &Ly.route_bias, (size_t)d.experts * 4));
            TRY(hy_alloc_mat(ctx, Ly.egu, d.experts * 2 * Ly.eff_pad, W, W));
            TRY(hy_alloc_mat(ctx, Ly.edown, d.experts * W, Ly.eff_pad, Ly.eff_pad));
            max_rz = std::max(max_rz, Ly.router.rows); max_top = std::max(max_top, d.top); max_eff = std::max(max_eff, Ly.eff_pad); max_e = std::max(max_e, d.experts);
        }
        if (h->depth) TRY(hy_alloc(ctx, &Ly.depth_mix, (size_t)(l + 2) * 4));
        if (h->side_dim > 0) {
            TRY(hy_alloc_mat(ctx, Ly.side_gate, h->side_dim, W, W));
            TRY(hy_alloc_mat(ctx, Ly.side_proj, W, h->side_dim, h->side_ld));
            TRY(hy_alloc(ctx, &Ly.side_norm, (size_t)W * 4));
        }
        slot = (slot + 63) & ~(size_t)63;
    }
    h->slot_floats = slot;
    TRY(hy_alloc(ctx, &h->slots, slot * h->n_seqs * 4));
    TRY(hy_alloc(ctx, &h->X, (size_t)S * mb * W * 4));
    TRY(hy_alloc(ctx, &h->h, (size_t)mb * W * es));
    TRY(hy_alloc(ctx, &h->proj, (size_t)mb * max_proj * 4));
    TRY(hy_alloc(ctx, &h->y, (size_t)HY_YPARTS * mb * W * 4));          // K-split partial sums of the output / down projections
    h->max_heads = max_heads;
    TRY(hy_alloc(ctx, &h->gates, (size_t)3 * mb * max_heads * 4));
    TRY(hy_alloc(ctx, &h->rowr, (size_t)2 * mb * 4));
    TRY(hy_alloc(ctx, &h->mixo, (size_t)mb * max_mix * es));
    TRY(hy_alloc(ctx, &h->conv, (size_t)mb * max_ch * 4));
    TRY(hy_alloc(ctx, &h->ssm_y, (size_t)mb * max_inner * 4));
    TRY(hy_alloc(ctx, &h->qa, (size_t)mb * max_hr * 4));
    TRY(hy_alloc(ctx, &h->oc, (size_t)mb * max_hr * 4));
    if (max_qr > 0) {
        TRY(hy_alloc(ctx, &h->cq, (size_t)mb * max_qr * es));
        TRY(hy_alloc(ctx, &h->qfull, (size_t)mb * max_qfull * 4));
    }
    if (max_kx > 0 && (mb > 8 || long_latent)) {          // latent attention, portions of many tokens (or cached rows too long for the latent-space form): expanded keys / values of one layer at a time
        TRY(hy_alloc(ctx, &h->kx, (size_t)C * max_kx * 4));
        TRY(hy_alloc(ctx, &h->vx, (size_t)C * max_vx * 4));
    }
    h->part_rows = std::max<size_t>(mb, 16 * 128);         // (token, split) pairs: a portion at one split, or 16 decode tokens at 128
    TRY(hy_alloc(ctx, &h->part_acc, h->part_rows * max_hdv * 4));
    TRY(hy_alloc(ctx, &h->part_ml, h->part_rows * max_heads * 2 * 4));
    if (h->depth) TRY(hy_alloc(ctx, &h->hist, (size_t)(desc->n_layers + 1) * mb * W * 4));
    if (h->side_dim > 0) {
        TRY(hy_alloc(ctx, &h->xb, (size_t)mb * W * es));
        TRY(hy_alloc(ctx, &h->side_z, (size_t)HY_ZSPLIT * mb * h->side_dim * 4));
        TRY(hy_alloc(ctx, &h->side_g, (size_t)mb * h->side_ld * es));
    }
    h->max_top = max_top;
    if (max_top > 0) {
        const size_t P = (size_t)mb * max_top;
        TRY(hy_alloc(ctx, &h->moe_z, (size_t)HY_ZSPLIT * mb * max_rz * 4));
        TRY(hy_alloc(ctx, &h->sgz, (size_t)mb * 4));
        TRY(hy_alloc(ctx, &h->wsel, P * 4));
        TRY(hy_alloc(ctx, &h->sel, P * 4));
        TRY(hy_alloc(ctx, &h->pair_row, P * 4));
        TRY(hy_alloc(ctx, &h->tiles, 3 * (P / HY_MOE_BM + max_e + 1) * 4));
        TRY(hy_alloc(ctx, &h->ntiles, 4));
        TRY(hy_alloc(ctx, &h->ea, P * W * es));
        TRY(hy_alloc(ctx, &h->eact, P * max_eff * es));
        TRY(hy_alloc(ctx, &h->eout, P * W * 4));
    }
    TRY(hy_alloc(ctx, &h->xw, (size_t)h->want_cap * W * es));
    TRY(hy_alloc(ctx, &h->logits, (size_t)h->want_cap * V * 4));
    ctx->logits = h->logits;
    if (desc->flags & GL3_FLAG_LAYER_TAPS) TRY(hy_alloc(ctx, &h->taps, (size_t)desc->n_layers * mb * W * 4));
    TRY(hy_alloc(ctx, &h->ones, (size_t)HY_MAX_STREAMS * 4));
    {
        float one[HY_MAX_STREAMS];
        for (float& v : one) v = 1.f;
        TRYHIP(hipMemcpy(h->ones, one, sizeof one, hipMemcpyHostToDevice));
    }
    // step record, wanted rows and token ids travel in one copy: [dyn 4 | want want_cap | tokens mb]
    TRY(hy_alloc(ctx, &h->dyn, (size_t)(4 + h->want_cap + mb) * 4));
    h->want = h->dyn + 4; h->tokens = h->want + h->want_cap;
    TRYHIP(hipHostMalloc((void**)&h->h_dyn, (size_t)(4 + h->want_cap + mb) * 4));
    h->h_want = h->h_dyn + 4; h->h_tokens = h->h_want + h->want_cap;
    TRYHIP(hipHostMalloc((void**)&h->h_logits, (size_t)h->want_cap * V * 4));
    TRYHIP(hipMalloc((void**)&ctx->argmax, (2 + 2 * AMX_WGS) * sizeof(int)));
    TRYHIP(hipMemset(ctx->argmax, 0, (2 + 2 * AMX_WGS) * sizeof(int)));
    TRYHIP(hipHostMalloc((void**)&ctx->h_argmax, sizeof(int)));
    TRYHIP(hipHostMalloc((void**)&ctx->h_dyn, 4 * sizeof(int)));          // the samplers' result words (gl3_sample.hip)
    {   // attention tiles above the 64 KB default of dynamic LDS
#define HY_LDS(RW, DVL) TRYHIP(hipFuncSetAttribute((const void*)hy_attn_kernel<RW, DVL>, hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024))
        HY_LDS(1, 1); HY_LDS(1, 2); HY_LDS(1, 4); HY_LDS(1, 8); HY_LDS(2, 1); HY_LDS(2, 2); HY_LDS(2, 4); HY_LDS(2, 8);
        HY_LDS(4, 1); HY_LDS(4, 2); HY_LDS(4, 4); HY_LDS(4, 8); HY_LDS(8, 1); HY_LDS(8, 2); HY_LDS(8, 4);
#undef HY_LDS
    }
    TRYHIP(hipDeviceSynchronize());
#undef TRY
#undef TRYHIP
    *out = ctx;
    return GL3_OK;
}

void gl3_hy_destroy(gl3_ctx* ctx) {
    gl3_hybrid_state* h = ctx->hy;
    if (!h) return;
    auto f = [](void* p) { if (p) hipFree(p); };
    auto hf = [](void* p) { if (p) hipHostFree(p); };
    f(h->emb.w); f(h->head.w); f(h->final_norm);
    for (auto& L : h->L) {
        f(L.proj.w); f(L.o.w); f(L.gu.w); f(L.down.w); f(L.norm1); f(L.norm2); f(L.pbias);
        for (auto& q : L.hc) for (float* p : q) f(p);
        for (HyLayer* M : {&L, L.side}) {
            if (!M) continue;
            f(M->lat_norm); f(M->wk); f(M->wv); f(M->wvT); f(M->conv_w); f(M->conv_b); f(M->dt_bias); f(M->a_log); f(M->dskip); f(M->ssm_norm);
            f(M->rot_freq); f(M->vrot_freq); f(M->qn); f(M->kn); f(M->sink); f(M->decay); f(M->uq.w); f(M->qlat_norm); f(M->lat_freq);
        }
        delete L.side;
        L.side = nullptr;
        f(L.norm1b); f(L.norm2b); f(L.route_bias);
        f(L.router.w); f(L.egu.w); f(L.edown.w); f(L.depth_mix); f(L.side_gate.w); f(L.side_proj.w); f(L.side_norm);
    }
    f(h->side_emb.w); f(h->sgz); f(h->hist); f(h->side_z); f(h->moe_z); f(h->wsel); f(h->eout); f(h->xb); f(h->side_g); f(h->ea); f(h->eact); f(h->sel); f(h->pair_row); f(h->tiles); f(h->ntiles);
    f(h->slots); f(h->X); f(h->h); f(h->proj); f(h->y); f(h->mixo); f(h->conv); f(h->ssm_y); f(h->qa); f(h->oc); f(h->kx); f(h->vx); f(h->part_acc); f(h->part_ml); f(h->gates); f(h->rowr);
    f(h->cq); f(h->qfull);
    f(h->xw); f(h->logits); f(h->taps); f(h->ones); f(h->dyn);
    hf(h->h_dyn); hf(h->h_logits);
    if (ctx->logits == h->logits) ctx->logits = nullptr;
    delete h;
    ctx->hy = nullptr;
}

// ---- upload -----------------------------------------------------------------------------------------------------------------------
static bool hy_to_f32(const void* host, uint64_t bytes, int type, size_t n, std::vector<float>& out) {
    out.resize(n);
    if (type == GL3_TYPE_BF16) {
        if (bytes != n * 2) return false;
        const uint16_t* s = (const uint16_t*)host;
        for (size_t i = 0; i < n; ++i) out[i] = hy_bf16_to_f32(s[i]);
    } else if (type == GL3_TYPE_F32) {
        if (bytes != n * 4) return false;
        memcpy(out.data(), host, bytes);
    } else
        return false;
    return true;
}
static int32_t hy_put_vec(gl3_ctx* ctx, float* dst, size_t n, const void* host, uint64_t bytes, int type, float add = 0.f) {
    std::vector<float> f;
    if (!hy_to_f32(host, bytes, type, n, f)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
    if (add != 0.f)
        for (float& v : f) v += add;
    HY_HIP(hipMemcpy(dst, f.data(), n * 4, hipMemcpyHostToDevice));
    return GL3_OK;
}
// rows x k source -> rows dst_row0 .., columns dst_col0 .. dst_col0 + k - 1 of m (the matrix's other columns keep what they hold).
// block32 = 1 / 2: source row r goes to row (r / 32) 64 + r % 32 (+ 32 for 2)
static int32_t hy_put_rows(gl3_ctx* ctx, HyMat& m, int dst_row0, int rows, int k, const void* host, uint64_t bytes, int type, int block32, int dst_col0 = 0) {
    const bool f32 = ctx->hy->f32;
    const size_t es = f32 ? 4 : 2, n = (size_t)rows * k;
    if ((type != GL3_TYPE_BF16 && type != GL3_TYPE_F32) || bytes != n * (type == GL3_TYPE_BF16 ? 2 : 4)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
    if (dst_col0 < 0 || dst_col0 + k > m.k) GL3_FAIL(GL3_E_ARG, "tensor row length mismatch");
    std::vector<uint8_t> img(n * es, 0);
    for (size_t i = 0; i < n; ++i) {
        if (f32) ((float*)img.data())[i] = type == GL3_TYPE_BF16 ? hy_bf16_to_f32(((const uint16_t*)host)[i]) : ((const float*)host)[i];
        else ((uint16_t*)img.data())[i] = type == GL3_TYPE_BF16 ? ((const uint16_t*)host)[i] : hy_f32_to_bf16(((const float*)host)[i]);
    }
    const size_t rb = (size_t)m.ld * es, sb = (size_t)k * es;
    uint8_t* base = (uint8_t*)m.w + (size_t)dst_col0 * es;
    if (!block32) {
        if (dst_row0 + rows > m.rows) GL3_FAIL(GL3_E_ARG, "tensor has too many rows");
        HY_HIP(hipMemcpy2D(base + (size_t)dst_row0 * rb, rb, img.data(), sb, sb, rows, hipMemcpyHostToDevice));
    } else {
        for (int r0 = 0; r0 < rows; r0 += 32) {
            const int nr = std::min(32, rows - r0), dr = dst_row0 + (r0 / 32) * 64 + (block32 == 2 ? 32 : 0);
            if (dr + nr > m.rows) GL3_FAIL(GL3_E_ARG, "tensor has too many rows");
            HY_HIP(hipMemcpy2D(base + (size_t)dr * rb, rb, img.data() + (size_t)r0 * sb, sb, sb, nr, hipMemcpyHostToDevice));
        }
    }
    return GL3_OK;
}

int32_t gl3_hy_upload(gl3_ctx* ctx, int32_t id, int32_t layer, const void* host, uint64_t bytes, int32_t type) {
    gl3_hybrid_state* h = ctx->hy;
    if (!host) GL3_FAIL(GL3_E_ARG, "null tensor data");
    if (id < 0 || id >= GL3_T_COUNT) GL3_FAIL(GL3_E_ARG, "unknown tensor id");
    HY_HIP(hipSetDevice(ctx->d.device));
    const int W = h->W, S = h->S;
    constexpr int32_t NOT_MINE = -1000;
    int32_t r = NOT_MINE;
    if (id == GL3_T_TOKEN_EMBD || id == GL3_T_OUTPUT || id == GL3_T_OUTPUT_NORM || id == GL3_T_SIDE_EMBD) {
        if (id == GL3_T_TOKEN_EMBD) r = hy_put_rows(ctx, h->emb, 0, ctx->d.vocab, W, host, bytes, type, 0);
        else if (id == GL3_T_OUTPUT) r = hy_put_rows(ctx, h->head, 0, ctx->d.vocab, W, host, bytes, type, 0);
        else if (id == GL3_T_SIDE_EMBD) {
            if (h->side_dim < 1) GL3_FAIL(GL3_E_ARG, "the model has no per-layer token input");
            r = hy_put_rows(ctx, h->side_emb, 0, ctx->d.vocab, h->side_emb.k, host, bytes, type, 0);
        } else r = hy_put_vec(ctx, h->final_norm, W, host, bytes, type, h->norm_offset);
        if (r == GL3_OK) h->have |= 1ull << id;
        return r;
    }
    const bool beside = layer >= 0 && (layer & GL3_LAYER_BESIDE);
    if (beside) layer &= ~GL3_LAYER_BESIDE;
    if (layer < 0 || layer >= (int)h->L.size()) GL3_FAIL(GL3_E_ARG, "layer out of range");
    HyLayer& L0 = h->L[layer];                       // the layer: its fused projection, output projection and feed-forward
    if (beside && !L0.side) GL3_FAIL(GL3_E_ARG, "layer " + std::to_string(layer) + " has no second mixer");
    HyLayer& L = beside ? *L0.side : L0;             // the mixer the tensor belongs to
    const gl3_layer_desc& d = L.d;
    const bool att = d.mixer == GL3_MIX_ATTENTION, lat = d.mixer == GL3_MIX_LATENT, ssm = d.mixer == GL3_MIX_SSM, mem = d.mixer == GL3_MIX_MEMORY;
    const bool memg = mem && d.mem_gates == GL3_MEM_EXP_GATES;
    const int mo = hy_mix_out(d);
    HyMat& proj = L0.proj;
    const size_t tes = type == GL3_TYPE_BF16 ? 2 : 4;          // bytes per element of the source
    std::vector<float> f;
    switch (id) {
        case GL3_T_ATTN_NORM: if (!beside) r = hy_put_vec(ctx, L.norm1, W, host, bytes, type, h->norm_offset); break;
        case GL3_T_FFN_NORM: if (d.ff > 0 && L.norm2) r = hy_put_vec(ctx, L.norm2, W, host, bytes, type, h->norm_offset); break;
        case GL3_T_ATTN_POST_NORM: if (!beside && L.norm1b) r = hy_put_vec(ctx, L.norm1b, W, host, bytes, type, h->norm_offset); break;
        case GL3_T_FFN_POST_NORM: if (!beside && L.norm2b) r = hy_put_vec(ctx, L.norm2b, W, host, bytes, type, h->norm_offset); break;
        case GL3_T_WQ:
            if (lat && d.q_rank > 0) r = hy_put_rows(ctx, L.uq, 0, d.heads * L.De, d.q_rank, host, bytes, type, 0);
            else if (lat) r = hy_put_rows(ctx, proj, L.q_off, d.heads * L.De, W, host, bytes, type, 0);
            else if (att || mem) r = hy_put_rows(ctx, proj, L.q_off, d.heads * d.dim, W, host, bytes, type, 0);
            break;
        case GL3_T_Q_DOWN: if (lat && d.q_rank > 0) r = hy_put_rows(ctx, proj, L.q_off, d.q_rank, W, host, bytes, type, 0); break;
        case GL3_T_Q_DOWN_NORM: if (lat && d.q_rank > 0) r = hy_put_vec(ctx, L.qlat_norm, d.q_rank, host, bytes, type); break;
        case GL3_T_FFN_ROUTE_BIAS: if (d.experts > 0 && d.route_bias) r = hy_put_vec(ctx, L.route_bias, d.experts, host, bytes, type); break;
        case GL3_T_WK: if (att || mem) r = hy_put_rows(ctx, proj, L.k_off, d.kv_heads * d.dim, W, host, bytes, type, 0); break;
        case GL3_T_WV: if (att || mem) r = hy_put_rows(ctx, proj, L.v_off, d.kv_heads * d.vdim, W, host, bytes, type, 0); break;
        case GL3_T_ATTN_GATE: if (((att || lat) && d.out_gate) || mem) r = hy_put_rows(ctx, proj, L.g_off, hy_gate_rows(d), W, host, bytes, type, 0); break;
        case GL3_T_WO: r = hy_put_rows(ctx, L0.o, 0, W, mo, host, bytes, type, 0, L.o0); break;
        case GL3_T_BQ: if (att && d.qk_bias) r = hy_put_vec(ctx, L.pbias + L.q_off, (size_t)d.heads * d.dim, host, bytes, type); break;
        case GL3_T_BK: if (att && d.qk_bias) r = hy_put_vec(ctx, L.pbias + L.k_off, (size_t)d.kv_heads * d.dim, host, bytes, type); break;
        case GL3_T_BV: if (att && d.qk_bias) r = hy_put_vec(ctx, L.pbias + L.v_off, (size_t)d.kv_heads * d.vdim, host, bytes, type); break;
        case GL3_T_ATTN_Q_NORM: if (att && d.qk_unit_norm == 2) r = hy_put_vec(ctx, L.qn, (size_t)d.heads * d.dim, host, bytes, type); break;
        case GL3_T_ATTN_K_NORM: if (att && d.qk_unit_norm == 2) r = hy_put_vec(ctx, L.kn, (size_t)d.kv_heads * d.dim, host, bytes, type); break;
        case GL3_T_ATTN_SINK: if (att && d.softmax_sink == 2) r = hy_put_vec(ctx, L.sink, d.heads, host, bytes, type); break;
        case GL3_T_MEM_IGATE: if (memg) r = hy_put_rows(ctx, proj, L.i_off, d.heads, W, host, bytes, type, 0); break;
        case GL3_T_MEM_FGATE: if (memg) r = hy_put_rows(ctx, proj, L.f_off, d.heads, W, host, bytes, type, 0); break;
        case GL3_T_MEM_IGATE_BIAS: if (memg) r = hy_put_vec(ctx, L.pbias + L.i_off, d.heads, host, bytes, type); break;
        case GL3_T_MEM_FGATE_BIAS: if (memg) r = hy_put_vec(ctx, L.pbias + L.f_off, d.heads, host, bytes, type); break;
        case GL3_T_KV_DOWN: if (lat && d.kv_share == 0) r = hy_put_rows(ctx, proj, L.c_off, L.Re, W, host, bytes, type, 0); break;
        case GL3_T_KV_DOWN_NORM: if (lat && d.kv_share == 0) r = hy_put_vec(ctx, L.lat_norm, d.kv_rank, host, bytes, type); break;
        case GL3_T_K_UP:
            if (lat) {          // [h][dim][kv_rank] -> [h][De][Re]: zeros behind the latent's columns, and the rotated entries pass (identity)
                const int R = d.kv_rank, De = L.De, Re = L.Re;
                if (!hy_to_f32(host, bytes, type, (size_t)d.heads * d.dim * R, f)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
                std::vector<float> wk((size_t)d.heads * De * Re, 0.f);
                for (int hh = 0; hh < d.heads; ++hh) {
                    for (int dd = 0; dd < d.dim; ++dd) memcpy(&wk[((size_t)hh * De + dd) * Re], &f[((size_t)hh * d.dim + dd) * R], (size_t)R * 4);
                    for (int j = 0; j < d.rot_dim; ++j) wk[((size_t)hh * De + d.dim + j) * Re + R + j] = 1.f;
                }
                HY_HIP(hipMemcpy(L.wk, wk.data(), wk.size() * 4, hipMemcpyHostToDevice));
                r = GL3_OK;
            }
            break;
        case GL3_T_V_UP:
            if (lat) {          // [h][v][kv_rank] -> [h][v][Re] (zeros behind the latent's columns) and its transpose [h][Re][v]
                const int R = d.kv_rank, Re = L.Re;
                const size_t n = (size_t)d.heads * d.vdim * Re;
                if (!hy_to_f32(host, bytes, type, (size_t)d.heads * d.vdim * R, f)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
                std::vector<float> wv(n, 0.f), tr(n, 0.f);
                for (int hh = 0; hh < d.heads; ++hh)
                    for (int v = 0; v < d.vdim; ++v)
                        for (int rr = 0; rr < R; ++rr) {
                            const float x = f[((size_t)hh * d.vdim + v) * R + rr];
                            wv[((size_t)hh * d.vdim + v) * Re + rr] = x;
                            tr[((size_t)hh * Re + rr) * d.vdim + v] = x;
                        }
                HY_HIP(hipMemcpy(L.wvT, tr.data(), n * 4, hipMemcpyHostToDevice));
                HY_HIP(hipMemcpy(L.wv, wv.data(), n * 4, hipMemcpyHostToDevice));
                r = GL3_OK;
            }
            break;
        case GL3_T_SSM_IN: if (ssm) r = hy_put_rows(ctx, proj, L.q_off, hy_proj_rows(d), W, host, bytes, type, 0); break;
        case GL3_T_SSM_CONV: if (ssm) r = hy_put_vec(ctx, L.conv_w, (size_t)hy_conv_ch(d) * d.conv, host, bytes, type); break;
        case GL3_T_SSM_CONV_BIAS: if (ssm) r = hy_put_vec(ctx, L.conv_b, hy_conv_ch(d), host, bytes, type); break;
        case GL3_T_SSM_DT_BIAS: if (ssm) r = hy_put_vec(ctx, L.dt_bias, d.heads, host, bytes, type); break;
        case GL3_T_SSM_A_LOG: if (ssm) r = hy_put_vec(ctx, L.a_log, d.heads, host, bytes, type); break;
        case GL3_T_SSM_D: if (ssm) r = hy_put_vec(ctx, L.dskip, d.heads, host, bytes, type); break;
        case GL3_T_SSM_NORM: if (ssm || (mem && d.mem_norm_weight)) r = hy_put_vec(ctx, L.ssm_norm, mo, host, bytes, type); break;
        case GL3_T_W1: if (L.dense_ff > 0 && (d.experts > 0 || d.ff_act != 2)) r = hy_put_rows(ctx, L.gu, 0, L.dense_ff, W, host, bytes, type, 1); break;
        case GL3_T_W3: if (L.dense_ff > 0) r = hy_put_rows(ctx, L.gu, 0, L.dense_ff, W, host, bytes, type, (d.experts == 0 && d.ff_act == 2) ? 0 : 2); break;
        case GL3_T_W2:
            if (L.dense_ff > 0) {          // [W][ff] into rows of ff_pad
                if (!hy_to_f32(host, bytes, type, (size_t)W * L.dense_ff, f)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
                std::vector<float> pad((size_t)W * L.ff_pad, 0.f);
                for (int rr = 0; rr < W; ++rr) memcpy(&pad[(size_t)rr * L.ff_pad], &f[(size_t)rr * L.dense_ff], (size_t)L.dense_ff * 4);
                r = hy_put_rows(ctx, L.down, 0, W, L.ff_pad, pad.data(), pad.size() * 4, GL3_TYPE_F32, 0);
            }
            break;
        // mixture of experts: router rows, then (one more row) the shared expert's gate; the experts' matrices arrive stacked [experts][..]
        case GL3_T_FFN_GATE_INP: if (d.experts > 0) r = hy_put_rows(ctx, L.router, 0, d.experts, W, host, bytes, type, 0); break;
        case GL3_T_FFN_GATE_INP_SHEXP: if (d.experts > 0 && d.shared_ff > 0 && !d.shared_ungated) r = hy_put_rows(ctx, L.router, d.experts, 1, W, host, bytes, type, 0); break;
        case GL3_T_FFN_GATE_EXPS: case GL3_T_FFN_UP_EXPS:
            if (d.experts > 0) {
                const size_t per = (size_t)d.ff * W * tes;
                if (bytes != per * d.experts) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
                for (int e = 0; e < d.experts; ++e) {
                    r = hy_put_rows(ctx, L.egu, e * 2 * L.eff_pad, d.ff, W, (const uint8_t*)host + e * per, per, type, id == GL3_T_FFN_GATE_EXPS ? 1 : 2);
                    if (r != GL3_OK) break;
                }
            }
            break;
        case GL3_T_FFN_DOWN_EXPS:
            if (d.experts > 0) {
                if (!hy_to_f32(host, bytes, type, (size_t)d.experts * W * d.ff, f)) GL3_FAIL(GL3_E_ARG, "tensor size or type mismatch");
                std::vector<float> pad((size_t)W * L.eff_pad, 0.f);
                for (int e = 0; e < d.experts; ++e) {
                    for (int rr = 0; rr < W; ++rr) memcpy(&pad[(size_t)rr * L.eff_pad], &f[((size_t)e * W + rr) * d.ff], (size_t)d.ff * 4);
                    r = hy_put_rows(ctx, L.edown, e * W, W, L.eff_pad, pad.data(), pad.size() * 4, GL3_TYPE_F32, 0);
                    if (r != GL3_OK) break;
                }
            }
            break;
        case GL3_T_DEPTH_MIX: if (h->depth) r = hy_put_vec(ctx, L.depth_mix, (size_t)layer + 2, host, bytes, type); break;
        case GL3_T_SIDE_GATE: if (h->side_dim > 0) r = hy_put_rows(ctx, L.side_gate, 0, h->side_dim, W, host, bytes, type, 0); break;
        case GL3_T_SIDE_PROJ: if (h->side_dim > 0) r = hy_put_rows(ctx, L.side_proj, 0, W, h->side_dim, host, bytes, type, 0); break;
        case GL3_T_SIDE_NORM: if (h->side_dim > 0) r = hy_put_vec(ctx, L.side_norm, W, host, bytes, type); break;
        case GL3_T_HC1_IN: case GL3_T_HC1_OUT: if (!h->plain) r = hy_put_vec(ctx, L.hc[0][id - GL3_T_HC1_IN], S, host, bytes, type); break;
        case GL3_T_HC1_MIX: if (!h->plain) r = hy_put_vec(ctx, L.hc[0][2], (size_t)S * S, host, bytes, type); break;
        case GL3_T_HC2_IN: case GL3_T_HC2_OUT: if (d.ff > 0 && !h->plain) r = hy_put_vec(ctx, L.hc[1][id - GL3_T_HC2_IN], S, host, bytes, type); break;
        case GL3_T_HC2_MIX: if (d.ff > 0 && !h->plain) r = hy_put_vec(ctx, L.hc[1][2], (size_t)S * S, host, bytes, type); break;
        default: break;
    }
    if (r == NOT_MINE) GL3_FAIL(GL3_E_ARG, "tensor id " + std::to_string(id) + " does not belong to layer " + std::to_string(layer));
    if (r == GL3_OK) L.have |= 1ull << id;
    return r;
}

// tensors of one mixer (second = the mixer beside the layer's first: it has no norm, tables or feed-forward of its own)
static uint64_t hy_needed(const gl3_hybrid_state* h, const gl3_layer_desc& d, bool second = false) {
    uint64_t m = 1ull << GL3_T_WO;
    if (d.mixer == GL3_MIX_ATTENTION) m |= (1ull << GL3_T_WQ) | (1ull << GL3_T_WK) | (1ull << GL3_T_WV);
    if (d.mixer == GL3_MIX_ATTENTION && d.qk_bias) m |= (1ull << GL3_T_BQ) | (1ull << GL3_T_BK) | (1ull << GL3_T_BV);
    if (d.mixer == GL3_MIX_ATTENTION && d.qk_unit_norm == 2) m |= (1ull << GL3_T_ATTN_Q_NORM) | (1ull << GL3_T_ATTN_K_NORM);
    if (d.mixer == GL3_MIX_ATTENTION && d.softmax_sink == 2) m |= 1ull << GL3_T_ATTN_SINK;
    if (d.mixer == GL3_MIX_MEMORY) m |= (1ull << GL3_T_WQ) | (1ull << GL3_T_WK) | (1ull << GL3_T_WV) | (1ull << GL3_T_ATTN_GATE);
    if (d.mixer == GL3_MIX_MEMORY && d.mem_norm_weight) m |= 1ull << GL3_T_SSM_NORM;
    if (d.mixer == GL3_MIX_MEMORY && d.mem_gates == GL3_MEM_EXP_GATES)
        m |= (1ull << GL3_T_MEM_IGATE) | (1ull << GL3_T_MEM_FGATE) | (1ull << GL3_T_MEM_IGATE_BIAS) | (1ull << GL3_T_MEM_FGATE_BIAS);
    if (second) return m;
    m |= 1ull << GL3_T_ATTN_NORM;
    if (!h->plain) m |= (1ull << GL3_T_HC1_IN) | (1ull << GL3_T_HC1_OUT) | (1ull << GL3_T_HC1_MIX);
    if (h->depth) m |= 1ull << GL3_T_DEPTH_MIX;
    if (h->side_dim > 0) m |= (1ull << GL3_T_SIDE_GATE) | (1ull << GL3_T_SIDE_PROJ) | (1ull << GL3_T_SIDE_NORM);
    if (d.mixer == GL3_MIX_LATENT) m |= (1ull << GL3_T_WQ) | (1ull << GL3_T_K_UP) | (1ull << GL3_T_V_UP);
    if (d.mixer == GL3_MIX_LATENT && d.kv_share == 0) m |= (1ull << GL3_T_KV_DOWN) | (1ull << GL3_T_KV_DOWN_NORM);
    if (d.mixer == GL3_MIX_LATENT && d.q_rank > 0) m |= (1ull << GL3_T_Q_DOWN) | (1ull << GL3_T_Q_DOWN_NORM);
    if (h->post_norms) m |= (1ull << GL3_T_ATTN_POST_NORM) | (d.ff > 0 ? 1ull << GL3_T_FFN_POST_NORM : 0);
    if (d.experts > 0 && d.route_bias) m |= 1ull << GL3_T_FFN_ROUTE_BIAS;
    if ((d.mixer == GL3_MIX_ATTENTION || d.mixer == GL3_MIX_LATENT) && d.out_gate) m |= 1ull << GL3_T_ATTN_GATE;
    if (d.mixer == GL3_MIX_SSM)
        m |= (1ull << GL3_T_SSM_IN) | (1ull << GL3_T_SSM_CONV) | (1ull << GL3_T_SSM_CONV_BIAS) | (1ull << GL3_T_SSM_DT_BIAS) | (1ull << GL3_T_SSM_A_LOG) |
             (1ull << GL3_T_SSM_D) | (1ull << GL3_T_SSM_NORM);
    if (d.ff > 0 && !h->parallel) m |= 1ull << GL3_T_FFN_NORM;
    if (d.ff > 0 && !h->plain) m |= (1ull << GL3_T_HC2_IN) | (1ull << GL3_T_HC2_OUT) | (1ull << GL3_T_HC2_MIX);
    if (d.experts > 0) m |= (1ull << GL3_T_FFN_GATE_INP) | (1ull << GL3_T_FFN_GATE_EXPS) | (1ull << GL3_T_FFN_UP_EXPS) | (1ull << GL3_T_FFN_DOWN_EXPS);
    if (d.experts > 0 && d.shared_ff > 0 && !d.shared_ungated) m |= 1ull << GL3_T_FFN_GATE_INP_SHEXP;
    if (d.experts > 0 ? d.shared_ff > 0 : d.ff > 0) m |= (1ull << GL3_T_W2) | (1ull << GL3_T_W3) | ((d.experts > 0 || d.ff_act != 2) ? 1ull << GL3_T_W1 : 0);
    return m;
}

int32_t gl3_hy_finalize(gl3_ctx* ctx) {
    gl3_hybrid_state* h = ctx->hy;
    const uint64_t g = (1ull << GL3_T_TOKEN_EMBD) | (1ull << GL3_T_OUTPUT_NORM) | (h->side_dim > 0 ? 1ull << GL3_T_SIDE_EMBD : 0);
    if ((h->have & g) != g) GL3_FAIL(GL3_E_STATE, "missing global tensors (token embedding / output norm / side embedding)");
    if (!(h->have & (1ull << GL3_T_OUTPUT))) {           // tied head
        HY_HIP(hipMemcpy(h->head.w, h->emb.w, (size_t)h->emb.rows * h->emb.ld * (h->f32 ? 4 : 2), hipMemcpyDeviceToDevice));
    }
    for (size_t l = 0; l < h->L.size(); ++l) {
        const uint64_t need = hy_needed(h, h->L[l].d);
        if ((h->L[l].have & need) != need) GL3_FAIL(GL3_E_STATE, "layer " + std::to_string(l) + ": missing tensors");
        if (h->L[l].side) {
            const uint64_t need2 = hy_needed(h, h->L[l].side->d, true);
            if ((h->L[l].side->have & need2) != need2) GL3_FAIL(GL3_E_STATE, "layer " + std::to_string(l) + ", second mixer: missing tensors");
        }
    }
    if (h->logit_mul != 1.f) {          // the logits' multiplier rides on the final norm's weight
        std::vector<float> w(h->W);
        HY_HIP(hipMemcpy(w.data(), h->final_norm, (size_t)h->W * 4, hipMemcpyDeviceToHost));
        for (float& v : w) v *= h->logit_mul;
        HY_HIP(hipMemcpy(h->final_norm, w.data(), (size_t)h->W * 4, hipMemcpyHostToDevice));
    }
    HY_HIP(hipDeviceSynchronize());
    ctx->finalized = true;
    return GL3_OK;
}

// ---- launches -----------------------------------------------------------------------------------------------------------------------
// activation of the layer's dense feed-forward (in a mixture of experts: of the shared expert)
static HyGlu hy_ff_glu(const HyLayer& L) { return HyGlu{L.dense_limit, L.d.ff_alpha, L.d.ff_shift, nullptr, nullptr, 0, 0, L.d.ff_act}; }
// parts != null: C has room for HY_KSPLIT copies and the caller sums them (the streams kernel does); *parts = copies written
template <typename T>
static void hy_gemm(gl3_ctx* ctx, const T* A, int lda, const HyMat& w, int M, float* C, int ldc, bool glu, T* act, int ld_act, HyGlu gp, int* parts = nullptr, int max_parts = HY_KSPLIT) {
    if (parts) *parts = 1;
    const T* Wt = (const T*)w.w;
    const int N = w.rows, K = w.k;
    hipStream_t st = ctx->stream;
    if (M <= 8) {
        const int pairs = hy_cdiv(N, 2);
        const bool ksplit = pairs < 8192 && K >= 1024;       // few rows: a workgroup's four wavefronts share one pair's K
        const int wgs = ksplit ? pairs : hy_cdiv(pairs, 4);
#define HY_MV2(MT, KS)                                                                                                                              \
    do {                                                                                                                                            \
        if (glu) hipLaunchKernelGGL((hy_matvec_kernel<T, T, MT, HY_EPI_GLU, KS>), dim3(wgs), dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp);   \
        else if (gp.mul_table || gp.act == 2) hipLaunchKernelGGL((hy_matvec_kernel<T, T, MT, HY_EPI_ACTMUL, KS>), dim3(wgs), dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp);   \
        else hipLaunchKernelGGL((hy_matvec_kernel<T, T, MT, HY_EPI_STORE, KS>), dim3(wgs), dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp);    \
    } while (0)
#define HY_MV(MT) do { if (ksplit) HY_MV2(MT, 4); else HY_MV2(MT, 1); } while (0)
        if (M == 1) HY_MV(1); else if (M == 2) HY_MV(2); else if (M <= 4) HY_MV(4); else HY_MV(8);
#undef HY_MV2
#undef HY_MV
        return;
    }
    const long tiles = (long)hy_cdiv(M, 128) * hy_cdiv(N, 128);
    const bool big = tiles >= 256 || (parts && tiles >= 64);
    constexpr int BKT = HyPiece<T>::N * HyPiece<T>::PPR;
    int ks = 1;                                              // few result tiles and a long K: split K over blockIdx.z, the caller adds the parts
    if (parts && !glu && !gp.mul_table && gp.act != 2 && tiles < 192 && K >= 16 * BKT) ks = (int)std::min<long>(max_parts, std::max<long>(1, 256 / tiles));
    const int kper = hy_cdiv(hy_cdiv(K, ks), BKT) * BKT;
    ks = hy_cdiv(K, kper);
    if (parts) *parts = ks;
#define HY_GM(BM)                                                                                                                                   \
    do {                                                                                                                                            \
        const dim3 grid(hy_cdiv(N, 128), hy_cdiv(M, BM), ks);                                                                                         \
        if (glu) hipLaunchKernelGGL((hy_gemm_kernel<T, T, BM, 128, HY_EPI_GLU>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp, kper);    \
        else if (gp.mul_table || gp.act == 2) hipLaunchKernelGGL((hy_gemm_kernel<T, T, BM, 128, HY_EPI_ACTMUL>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp, kper);    \
        else hipLaunchKernelGGL((hy_gemm_kernel<T, T, BM, 128, HY_EPI_STORE>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, M, N, K, C, ldc, act, ld_act, gp, kper);     \
    } while (0)
    if (big) HY_GM(128); else HY_GM(64);
#undef HY_GM
}

// the streams kernel: 1024 threads per token for a few tokens, 256 for many
template <typename T>
static void hy_streams(gl3_ctx* ctx, int blocks, float* X, int W, int S, size_t sstride, const float* y, int yparts, size_t ystride, const float* post_mix, const float* post_out, const float* pre_in,
                       const float* norm_w, float eps, T* h_out, float* sum_out, const int* rows) {
    if (blocks <= 32)
        hipLaunchKernelGGL((hy_streams_kernel<T, 1024>), dim3(blocks), dim3(1024), 0, ctx->stream, X, W, S, sstride, y, yparts, ystride, post_mix, post_out, pre_in, norm_w, eps, h_out, sum_out, rows);
    else
        hipLaunchKernelGGL((hy_streams_kernel<T, 256>), dim3(blocks), dim3(256), 0, ctx->stream, X, W, S, sstride, y, yparts, ystride, post_mix, post_out, pre_in, norm_w, eps, h_out, sum_out, rows);
}

struct HyAttnPlan { int rw, dvl, kt; size_t smem; };
static HyAttnPlan hy_attn_plan(int rows, int dk, int dv, bool shared_kv) {
    HyAttnPlan p;
    const int c = hy_cdiv(dv, 64);
    p.dvl = c <= 1 ? 1 : c <= 2 ? 2 : c <= 4 ? 4 : 8;
    // rows per wavefront: 8 (4 with 512 value columns: RW x DVL accumulators per lane), fewer when the key / value head has few rows
    p.rw = p.dvl == 8 ? 4 : 8;
    while (p.rw > 1 && rows < 4 * p.rw) p.rw /= 2;
    // 8 rows only where two workgroups still share a CU's LDS with 64-key tiles
    if (p.rw == 8 && ((size_t)HY_KT * (dk | 1) + (shared_kv ? 0 : (size_t)HY_KT * dv) + 4 * (size_t)dk * 8 + 4 * (size_t)HY_KT * 8) * 4 > 80 * 1024) p.rw = 4;
    // diagnostic switches (read once): GL3_HY_ATTN_RW = rows per wavefront, GL3_HY_ATTN_KT = key rows per tile, for portions of many rows
    static const int env_rw = getenv("GL3_HY_ATTN_RW") ? atoi(getenv("GL3_HY_ATTN_RW")) : 0;
    static const int env_kt = getenv("GL3_HY_ATTN_KT") ? atoi(getenv("GL3_HY_ATTN_KT")) : 0;
    if (rows >= 64 && (env_rw == 1 || env_rw == 2 || env_rw == 4 || (env_rw == 8 && p.dvl < 8))) p.rw = env_rw;
    auto need = [&](int kt, int rw) { return ((size_t)kt * (dk | 1) + (shared_kv ? 0 : (size_t)kt * dv) + 4 * (size_t)dk * rw + 4 * (size_t)kt * rw) * 4; };
    while (p.rw > 1 && need(8, p.rw) > 120 * 1024) p.rw /= 2;          // very long keys: fewer rows per wavefront before the tile shrinks to nothing
    for (p.kt = (rows >= 64 && (env_kt == 8 || env_kt == 16 || env_kt == 32)) ? env_kt : HY_KT;; p.kt /= 2) {        // the largest key tile whose rows fit beside the queries (two workgroups per CU while 64 rows allow it)
        p.smem = ((size_t)p.kt * (dk | 1) + (shared_kv ? 0 : (size_t)p.kt * dv) + 4 * (size_t)dk * p.rw + 4 * (size_t)p.kt * p.rw) * 4;
        if (p.smem <= 120 * 1024 || p.kt == 8) break;
    }
    return p;
}

static int32_t hy_attention(gl3_ctx* ctx, const float* q, int ldq, const float* kc, const float* vc, int H, int G, int dk, int dv, float scale, float slope_log2,
                            int n, int pos0, int* nsplit_out, bool in_slot = true, int window = 0, int keep = 0, const float* pk = nullptr, const float* pv = nullptr, int pool = 0) {
    gl3_hybrid_state* h = ctx->hy;
    const bool shared_kv = kc == vc && dk == dv;
    HyAttnPlan p = hy_attn_plan(n * (H / G), dk, dv, shared_kv);
    if (p.smem > 150 * 1024) GL3_FAIL(GL3_E_UNSUPPORTED, "attention: key + value row too large for the LDS tile");
    int nsplit = 1;                                          // few tokens: one key tile per split while that gives <= 128 splits
    if (n <= 16) {
        int tiles = hy_cdiv(pos0 + n, p.kt);
        if (window > 0) tiles = std::min<long>(tiles, hy_cdiv(keep, p.kt) + ((long)window + n) / p.kt + 2);      // kept first keys + the window's tiles
        if (pool > 0) tiles += hy_cdiv(std::max(0, pos0 + n - window) / pool, p.kt);                               // + the tiles of pooled rows
        nsplit = std::min(128, std::max(1, tiles));
    }
    if ((size_t)n * nsplit > h->part_rows) nsplit = std::max<size_t>(1, h->part_rows / n);
    HyAttnArgs a;
    a.q = q; a.ldq = ldq; a.kc = kc; a.vc = vc; a.slot_stride = in_slot ? h->slot_floats : 0; a.H = H; a.G = G; a.dk = dk; a.dv = dv; a.scale = scale; a.slope_log2 = slope_log2;
    a.dyn = h->dyn; a.n = n; a.nsplit = nsplit; a.part_acc = h->part_acc; a.part_ml = h->part_ml; a.kt = p.kt; a.shared_kv = shared_kv ? 1 : 0; a.window = window; a.keep = keep;
    a.pk = pk; a.pv = pv; a.pool = pool;
    const dim3 grid((unsigned)hy_cdiv(n * (H / G), 4 * p.rw) * G, 1, nsplit);
#define HY_AT(RW, DVL) hipLaunchKernelGGL((hy_attn_kernel<RW, DVL>), grid, dim3(256), p.smem, ctx->stream, a)
#define HY_AT_RW(RW) do { if (p.dvl == 1) HY_AT(RW, 1); else if (p.dvl == 2) HY_AT(RW, 2); else if (p.dvl == 4) HY_AT(RW, 4); else HY_AT(RW, 8); } while (0)
    if (p.rw == 8) { if (p.dvl == 1) HY_AT(8, 1); else if (p.dvl == 2) HY_AT(8, 2); else HY_AT(8, 4); }
    else if (p.rw == 4) HY_AT_RW(4); else if (p.rw == 2) HY_AT_RW(2); else HY_AT_RW(1);
#undef HY_AT_RW
#undef HY_AT
    *nsplit_out = nsplit;
    return GL3_OK;
}

// The recurrence kernel: a column's states over NG lanes x NL registers: NL = 16 (32 for more than 1024 states, 8 / 4 for very small
// ones), NG a power of two; tokens staged per round: what fits 48 KB of LDS, at most 32.  Fills in a.NG and a.TB.
// With few workgroups (few heads, narrow values) NL = 16 is halved once so that more of them share the columns; below 8 every workgroup
// stages the same key / query rows for too few columns and the traffic from L2 eats the gain (measured: 16 and 8 within 2 %, 4 slower).
// GL3_HY_SCAN_NL forces a value.
static void hy_scan(gl3_ctx* ctx, HyScanArgs& a) {
    int NL = a.N > 1024 ? 32 : a.N > 8 ? 16 : a.N > 4 ? 8 : 4;
    auto wgs = [&](int nl) { int ng = 1; while (ng * nl < a.N) ng *= 2; return (long)hy_cdiv(a.P, 4 * (64 / ng)) * a.heads; };
    if (NL == 16 && 8 * 64 >= a.N && wgs(16) < 512) NL = 8;
    static const int env_nl = getenv("GL3_HY_SCAN_NL") ? atoi(getenv("GL3_HY_SCAN_NL")) : 0;
    if ((env_nl == 4 || env_nl == 8 || env_nl == 16 || env_nl == 32) && env_nl * 64 >= a.N) NL = env_nl;
    int NG = 1;
    while (NG * NL < a.N) NG *= 2;
    const int cols = 4 * (64 / NG), Ns = NG * NL;
    int TB = (int)(48 * 1024 / ((2 * (size_t)Ns + cols + 258) * 4));
    TB = std::max(1, std::min(32, TB));
    const size_t smem = ((size_t)TB * (2 * Ns + cols + 256) + 2 * TB) * 4;
    a.NG = NG; a.TB = TB;
    const dim3 grid(hy_cdiv(a.P, cols), a.heads);
#define HY_SCAN(NLT) hipLaunchKernelGGL((hy_ssm_scan_kernel<NLT>), grid, dim3(256), smem, ctx->stream, a)
    if (NL == 4) HY_SCAN(4); else if (NL == 8) HY_SCAN(8); else if (NL == 16) HY_SCAN(16); else HY_SCAN(32);
#undef HY_SCAN
}

// One mixer of a layer on the n rows of the fused projection in h->proj (row stride np): its heads land in mixo (row stride ldo) from
// column L.o0 on, multiplied by L.out_mul.
template <typename T>
static int32_t hy_mixer_core(gl3_ctx* ctx, HyLayer& L, int np, int ldo, int n, int pos0, int seq) {
    gl3_hybrid_state* h = ctx->hy;
    const gl3_layer_desc& d = L.d;
    hipStream_t st = ctx->stream;
    const float eps = ctx->d.rms_eps;
    T* mixo = (T*)h->mixo + L.o0;
    int nsplit = 1;
    if (d.mixer == GL3_MIX_ATTENTION) {
        float* kc = h->slots + L.off_k;
        float* vc = h->slots + L.off_v;
        float* pk = d.pool > 0 ? h->slots + L.off_pk : nullptr;
        float* pv = d.pool > 0 ? h->slots + L.off_pv : nullptr;
        const HyRot rot{d.rot_dims, L.rot_freq, d.v_unit_norm, d.v_rot ? L.vrot_freq : nullptr, d.rot_interleaved};
        const HyPrepX px{d.qk_bias ? L.pbias : nullptr, L.qn, L.kn, h->rowr};
        if (d.qk_unit_norm == 2) {
            if (n <= 32) hipLaunchKernelGGL((hy_rowrms_kernel<1024>), dim3(n, 2), dim3(1024), 0, st, h->proj, np, L.q_off, d.heads * d.dim, L.k_off, d.kv_heads * d.dim, px.bias, eps, h->rowr);
            else hipLaunchKernelGGL((hy_rowrms_kernel<256>), dim3(n, 2), dim3(256), 0, st, h->proj, np, L.q_off, d.heads * d.dim, L.k_off, d.kv_heads * d.dim, px.bias, eps, h->rowr);
        }
        hipLaunchKernelGGL(hy_attn_prep_kernel, dim3(n, d.heads + 2 * d.kv_heads), dim3(64), 0, st, h->proj, np, L.q_off, L.k_off, L.v_off, d.heads, d.kv_heads, d.dim,
                           d.vdim, d.qk_unit_norm, eps, kc, vc, h->slot_floats, h->dyn, rot, px);
        if (d.pool > 0) {
            const int done = (pos0 + n) / d.pool - pos0 / d.pool;          // blocks whose last position lies in this portion
            if (done > 0)
                hipLaunchKernelGGL(hy_pool_kernel, dim3(done, 2, done <= 8 ? std::min(16, hy_cdiv(d.kv_heads * std::max(d.dim, d.vdim), 256)) : 1), dim3(256), 0, st, kc, vc, pk, pv,
                                   d.kv_heads * d.dim, d.kv_heads * d.vdim, d.pool, h->slot_floats, h->dyn, n);
        }
        int32_t r = hy_attention(ctx, h->proj + L.q_off, np, kc, vc, d.heads, d.kv_heads, d.dim, d.vdim, d.scale, d.slope_log2, n, pos0, &nsplit, true, d.window, d.keep_first,
                                 pk, pv, d.pool);
        if (r != GL3_OK) return r;
        hipLaunchKernelGGL((hy_attn_merge_kernel<T>), dim3(n, d.heads), dim3(64), 0, st, h->part_acc, h->part_ml, d.heads, d.vdim, nsplit, d.softmax_sink,
                           d.out_gate ? h->proj + L.g_off : nullptr, np, d.out_gate, mixo, ldo, d.v_rot ? L.vrot_freq : nullptr, h->dyn,
                           d.softmax_sink == 2 ? L.sink : nullptr, L.out_mul);
    } else if (d.mixer == GL3_MIX_MEMORY) {
        const bool eg = d.mem_gates == GL3_MEM_EXP_GATES;
        const int P = d.vdim + (eg ? 1 : 0), ldy = d.heads * P;
        float *ga = h->gates, *gb = ga + (size_t)h->mb * h->max_heads, *ge = gb + (size_t)h->mb * h->max_heads;
        if (eg)
            hipLaunchKernelGGL(hy_mem_gates_kernel, dim3(d.heads), dim3(256), 0, st, h->proj, np, L.i_off, L.f_off, L.pbias, d.mem_gate_cap, d.heads, h->slots + L.off_m,
                               h->slot_floats, h->dyn, n, ga, gb, ge);
        HyScanArgs a{};
        a.ksrc = h->proj; a.ldk = np; a.k_off = L.k_off; a.k_hstride = d.dim;
        a.qsrc = h->proj; a.ldq = np; a.q_off = L.q_off; a.q_hstride = d.dim;
        a.xsrc = h->proj; a.ldx = np; a.x_off = L.v_off;
        a.k_mul = d.mem_k_mul != 0.f ? d.mem_k_mul : 1.f; a.q_mul = d.mem_q_mul != 0.f ? d.mem_q_mul : 1.f;
        a.act = d.mem_qkv_act;
        a.rot = HyScanRot{d.rot_dims, L.rot_freq, d.rot_interleaved};
        a.mode = eg ? 1 : 2; a.ga = ga; a.gb = gb; a.decay = L.decay; a.ones_col = eg ? 1 : 0;
        a.heads = d.heads; a.P = P; a.N = d.dim; a.G = d.heads;
        a.state = h->slots + L.off_state; a.slot_stride = h->slot_floats; a.dyn = h->dyn; a.n = n; a.y = h->ssm_y; a.ldy = ldy;
        hy_scan(ctx, a);
        if (d.mem_norm_whole && !eg) {          // one norm over the heads side by side: the kernel's "head" is the token's whole row
            // (a row is heads x vdim wide: 1024 threads for a few tokens, 256 for many)
            if (n <= 32 && ldy > 512)
                hipLaunchKernelGGL((hy_mem_out_kernel<T, 1024>), dim3(n, 1), dim3(1024), 0, st, h->ssm_y, ldy, ldy, ldy, (const float*)nullptr, 1,
                                   d.mem_norm_weight ? L.ssm_norm : nullptr, h->proj, np, L.g_off, d.mem_gate_act, eps, L.out_mul, mixo, ldo);
            else if (ldy > 128)
                hipLaunchKernelGGL((hy_mem_out_kernel<T, 256>), dim3(n, 1), dim3(256), 0, st, h->ssm_y, ldy, ldy, ldy, (const float*)nullptr, 1,
                                   d.mem_norm_weight ? L.ssm_norm : nullptr, h->proj, np, L.g_off, d.mem_gate_act, eps, L.out_mul, mixo, ldo);
            else
                hipLaunchKernelGGL((hy_mem_out_kernel<T, 64>), dim3(n, 1), dim3(64), 0, st, h->ssm_y, ldy, ldy, ldy, (const float*)nullptr, 1,
                                   d.mem_norm_weight ? L.ssm_norm : nullptr, h->proj, np, L.g_off, d.mem_gate_act, eps, L.out_mul, mixo, ldo);
        } else if (n <= 32 && d.vdim > 128)
            hipLaunchKernelGGL((hy_mem_out_kernel<T, 256>), dim3(n, d.heads), dim3(256), 0, st, h->ssm_y, ldy, P, d.vdim, eg ? ge : nullptr, d.heads,
                               d.mem_norm_weight ? L.ssm_norm : nullptr, h->proj, np, L.g_off, d.mem_gate_act, eps, L.out_mul, mixo, ldo);
        else
            hipLaunchKernelGGL((hy_mem_out_kernel<T, 64>), dim3(n, d.heads), dim3(64), 0, st, h->ssm_y, ldy, P, d.vdim, eg ? ge : nullptr, d.heads,
                               d.mem_norm_weight ? L.ssm_norm : nullptr, h->proj, np, L.g_off, d.mem_gate_act, eps, L.out_mul, mixo, ldo);
    } else if (d.mixer == GL3_MIX_LATENT) {
        // De entries per query / key head, Re per cached row (= dim, kv_rank without a rotated part)
        float* cc = h->slots + L.off_k;
        const int R = L.Re, De = L.De;
        float* q = h->proj + L.q_off;
        int ldq = np;
        if (d.q_rank > 0) {          // queries through their own latent: norm with weight, then the expansion
            hipLaunchKernelGGL((hy_rownorm_kernel<T>), dim3(n), dim3(256), 0, st, h->proj, np, L.q_off, d.q_rank, L.qlat_norm, eps, (T*)h->cq, d.q_rank);
            q = h->qfull; ldq = d.heads * De;
            hy_gemm<T>(ctx, (const T*)h->cq, d.q_rank, L.uq, n, q, ldq, false, nullptr, 0, HyGlu{});
        }
        if (d.rot_dim > 0)
            hipLaunchKernelGGL(hy_latent_prep_kernel, dim3(n, 1 + d.heads), dim3(64), 0, st, q, ldq, d.dim, d.rot_dim, h->proj, np, L.c_off, d.kv_rank, L.lat_norm, eps,
                               d.kv_share > 0 ? (float*)nullptr : cc, h->slot_floats, h->dyn, L.lat_freq, L.rot_mscale);
        else if (d.kv_share == 0)
            hipLaunchKernelGGL(hy_latent_norm_kernel, dim3(n), dim3(64), 0, st, h->proj, np, L.c_off, R, L.lat_norm, eps, cc, h->slot_floats, h->dyn);
        if (n > 8 || R > HY_LATENT_DIRECT) {
            // A portion of many tokens (or cached rows longer than the latent-space form below holds in registers): keys and values of every position so far are expanded from the slot's latents by two float32 GEMMs
            // into plan scratch (nothing but the latent is kept), and the attention core runs over them with one key / value head per
            // query head: 4 x less arithmetic than scoring in the latent's space when kv_rank is 4 x the head size.
            const int M = pos0 + n;
            const float* lat = cc + (size_t)seq * h->slot_floats;
            HyMat wkm, wvm;
            wkm.w = L.wk; wkm.rows = d.heads * De; wkm.k = R; wkm.ld = R;
            wvm.w = L.wv; wvm.rows = d.heads * d.vdim; wvm.k = R; wvm.ld = R;
            hy_gemm<float>(ctx, lat, R, wkm, M, h->kx, d.heads * De, false, nullptr, 0, HyGlu{});
            hy_gemm<float>(ctx, lat, R, wvm, M, h->vx, d.heads * d.vdim, false, nullptr, 0, HyGlu{});
            int32_t r = hy_attention(ctx, q, ldq, h->kx, h->vx, d.heads, d.heads, De, d.vdim, d.scale, 0.f, n, pos0, &nsplit, false);
            if (r != GL3_OK) return r;
            hipLaunchKernelGGL((hy_attn_merge_kernel<T>), dim3(n, d.heads), dim3(64), 0, st, h->part_acc, h->part_ml, d.heads, d.vdim, nsplit, d.softmax_sink,
                               d.out_gate ? h->proj + L.g_off : nullptr, np, d.out_gate == 2 ? 2 : 1, mixo, ldo, (const float*)nullptr, h->dyn);
        } else {
            // A few tokens (decode): the query is carried into the latent's space and the attention core reads the latents themselves
            // (one shared key / value head, keys = values), then the weighted sum of latents is expanded.
            if (n == 1)
                hipLaunchKernelGGL((hy_headmm_kernel<float, 1>), dim3(1, d.heads, hy_cdiv(R, 64)), dim3(256), 0, st, q, ldq, De, R, L.wk,
                                   (const float*)nullptr, 0, h->qa, d.heads * R, n);
            else
                hipLaunchKernelGGL((hy_headmm_kernel<float, 8>), dim3(hy_cdiv(n, 8), d.heads, hy_cdiv(R, 64)), dim3(256), 0, st, q, ldq, De, R, L.wk,
                                   (const float*)nullptr, 0, h->qa, d.heads * R, n);
            int32_t r = hy_attention(ctx, h->qa, d.heads * R, cc, cc, d.heads, 1, R, R, d.scale, 0.f, n, pos0, &nsplit);
            if (r != GL3_OK) return r;
            hipLaunchKernelGGL((hy_attn_merge_kernel<float>), dim3(n, d.heads), dim3(64), 0, st, h->part_acc, h->part_ml, d.heads, R, nsplit, d.softmax_sink,
                               (const float*)nullptr, 0, 0, h->oc, d.heads * R, (const float*)nullptr, h->dyn);
            if (n == 1)
                hipLaunchKernelGGL((hy_headmm_kernel<T, 1>), dim3(1, d.heads, hy_cdiv(d.vdim, 64)), dim3(256), 0, st, h->oc, d.heads * R, R, d.vdim, L.wvT,
                                   d.out_gate ? h->proj + L.g_off : nullptr, np, mixo, ldo, n, d.out_gate == 2 ? 2 : 1);
            else
                hipLaunchKernelGGL((hy_headmm_kernel<T, 8>), dim3(hy_cdiv(n, 8), d.heads, hy_cdiv(d.vdim, 64)), dim3(256), 0, st, h->oc, d.heads * R, R, d.vdim, L.wvT,
                                   d.out_gate ? h->proj + L.g_off : nullptr, np, mixo, ldo, n, d.out_gate == 2 ? 2 : 1);
        }
    } else {
        const int inner = d.heads * d.vdim, ch = hy_conv_ch(d), dt_off = 2 * inner + 2 * d.groups * d.state;
        float* state = h->slots + L.off_state;
        float* tail = h->slots + L.off_tail;
        hipLaunchKernelGGL(hy_conv_kernel, dim3(hy_cdiv(ch, 256), n), dim3(256), 0, st, h->proj, np, inner, ch, d.conv, L.conv_w, L.conv_b, tail, h->slot_floats, h->dyn,
                           n, h->conv);
        if (d.conv > 1)
            hipLaunchKernelGGL(hy_conv_tail_kernel, dim3(hy_cdiv(ch, 256)), dim3(256), 0, st, h->proj, np, inner, ch, d.conv, tail, h->slot_floats, h->dyn, n);
        HyScanArgs a{};
        a.ksrc = h->conv; a.ldk = ch; a.k_off = inner; a.k_hstride = d.state;
        a.qsrc = h->conv; a.ldq = ch; a.q_off = inner + d.groups * d.state; a.q_hstride = d.state;
        a.xsrc = h->conv; a.ldx = ch; a.x_off = 0;
        a.k_mul = a.q_mul = 1.f;
        a.mode = 0; a.dtsrc = h->proj; a.ld_dt = np; a.dt_off = dt_off; a.dt_bias = L.dt_bias; a.A_log = L.a_log; a.Dp = L.dskip;
        a.heads = d.heads; a.P = d.vdim; a.N = d.state; a.G = d.groups;
        a.state = state; a.slot_stride = h->slot_floats; a.dyn = h->dyn; a.n = n; a.y = h->ssm_y; a.ldy = inner;
        hy_scan(ctx, a);
        hipLaunchKernelGGL((hy_gated_norm_kernel<T>), dim3(n, d.norm_groups), dim3(256), 0, st, h->ssm_y, h->proj, np, 0, inner, d.norm_groups, L.ssm_norm, eps, mixo, ldo);
    }
    return GL3_OK;
}

// The mixer sublayer of a layer on the n normed rows in h->h: one product for the inputs of every mixer of the layer, the mixers'
// kernels, one product for their outputs (K-split parts in h->y, h->y_parts of them).
template <typename T>
static int32_t hy_mixer(gl3_ctx* ctx, HyLayer& L, int n, int pos0, int seq) {
    gl3_hybrid_state* h = ctx->hy;
    const int np = L.proj.rows;
    if (hy_narrow_proj(L.d) && !L.side) {
        // few result columns and a long K (a latent layer whose queries have their own latent): K-split parts, summed in place — the
        // mixer's kernels read single entries of the row
        int parts = 1;
        hy_gemm<T>(ctx, (T*)h->h, h->W, L.proj, n, h->proj, np, false, nullptr, 0, HyGlu{}, &parts);
        if (parts > 1) {
            const size_t cnt = (size_t)n * np;
            hipLaunchKernelGGL(hy_sum_parts_kernel, dim3((unsigned)std::min<size_t>(2048, (cnt + 1023) / 1024)), dim3(256), 0, ctx->stream, h->proj, parts, cnt, cnt);
        }
    } else
        hy_gemm<T>(ctx, (T*)h->h, h->W, L.proj, n, h->proj, np, false, nullptr, 0, HyGlu{});
    int32_t r = hy_mixer_core<T>(ctx, L, np, L.mo_total, n, pos0, seq);
    if (r == GL3_OK && L.side) r = hy_mixer_core<T>(ctx, *L.side, np, L.mo_total, n, pos0, seq);
    if (r != GL3_OK) return r;
    hy_gemm<T>(ctx, (T*)h->mixo, L.o.k, L.o, n, h->y, h->W, false, nullptr, 0, HyGlu{}, &h->y_parts);
    return GL3_OK;
}

// ---- mixture of experts -------------------------------------------------------------------------------------------------------------
// One product of every (token, choice) pair with its expert's matrix: w = ONE expert's shape (rows, k, ld) at the base of the stacked
// matrix, wstride elements apart.  few = a few tokens (decode): pairs in their own order, one matvec per pair (blockIdx.y) with the
// expert read from h->sel; else the pairs ordered by expert (h->tiles) and one MFMA tile per HY_MOE_BM rows of an expert.
template <typename T>
static void hy_gemm_grouped(gl3_ctx* ctx, const T* A, int lda, const HyMat& w, size_t wstride, int P, int max_tiles, bool few, float* C, int ldc, bool glu, T* act, int ld_act, HyGlu gp,
                            int a_div = 1, const float* row_scale = nullptr) {
    gl3_hybrid_state* h = ctx->hy;
    const T* Wt = (const T*)w.w;
    const int N = w.rows, K = w.k;
    hipStream_t st = ctx->stream;
    if (few) {
        const int pairs = hy_cdiv(N, 2);
        const bool ksplit = (long)pairs * P < 8192 && K >= 1024;
        const dim3 grid(ksplit ? pairs : hy_cdiv(pairs, 4), P);
#define HY_GMV(KS)                                                                                                                                     \
    do {                                                                                                                                              \
        if (glu) hipLaunchKernelGGL((hy_matvec_kernel<T, T, 1, HY_EPI_GLU, KS, 1>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, 1, N, K, C, ldc, act, ld_act, gp, h->sel, wstride, a_div, row_scale);   \
        else hipLaunchKernelGGL((hy_matvec_kernel<T, T, 1, HY_EPI_STORE, KS, 1>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, 1, N, K, C, ldc, act, ld_act, gp, h->sel, wstride, a_div, row_scale);    \
    } while (0)
        if (ksplit) HY_GMV(4); else HY_GMV(1);
#undef HY_GMV
        return;
    }
    const HyGroup grp{h->tiles, h->ntiles, wstride};
    const dim3 grid(hy_cdiv(N, 128), max_tiles, 1);
    if (glu) hipLaunchKernelGGL((hy_gemm_kernel<T, T, HY_MOE_BM, 128, HY_EPI_GLU, 1>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, 0, N, K, C, ldc, act, ld_act, gp, K, grp);
    else hipLaunchKernelGGL((hy_gemm_kernel<T, T, HY_MOE_BM, 128, HY_EPI_STORE, 1>), grid, dim3(256), 0, st, A, lda, Wt, w.ld, 0, N, K, C, ldc, act, ld_act, gp, K, grp);
}

// The feed-forward sublayer of a mixture-of-experts layer on the n normed rows in h->h: the routed experts' outputs land in h->eout (row
// h->pair_row[t top + k] for choice k of token t), the shared expert's in h->y (K-split parts), its gate's logit in h->moe_z[t][experts].
template <typename T>
static void hy_moe(gl3_ctx* ctx, HyLayer& L, int n) {
    gl3_hybrid_state* h = ctx->hy;
    const gl3_layer_desc& d = L.d;
    hipStream_t st = ctx->stream;
    const int W = h->W, E = d.experts, top = d.top, P = n * top, RZ = L.router.rows;
    T* hb = (T*)h->h;
    int zparts = 1;          // few result rows and a long K: the router's product comes in K-split parts that the route kernel adds
    hy_gemm<T>(ctx, hb, W, L.router, n, h->moe_z, RZ, false, nullptr, 0, HyGlu{}, &zparts, HY_ZSPLIT);
    const bool few = n <= 8;
    const int max_tiles = P / HY_MOE_BM + std::min(E, P);
    const bool on_out = d.route_on_output != 0;          // the weights multiply the experts' outputs (in the residual update) instead of their inputs
    hipLaunchKernelGGL(hy_route_kernel, dim3(n), dim3(64), 0, st, h->moe_z, RZ, zparts, (size_t)n * RZ, E, top, h->sel, h->wsel, few ? h->pair_row : nullptr,
                       (d.shared_ff > 0 && !d.shared_ungated) ? h->sgz : nullptr, HyRoute{d.route_softmax, L.route_bias, d.route_renorm, d.route_scale != 0.f ? d.route_scale : 1.f});
    HyMat one_gu = L.egu, one_down = L.edown;
    one_gu.rows = 2 * L.eff_pad; one_down.rows = W;
    if (few) {
        // a few tokens: the pairs of a token read its normed row themselves and the score multiplies the products (W (s h) = s (W h))
        hy_gemm_grouped<T>(ctx, hb, W, one_gu, (size_t)2 * L.eff_pad * L.egu.ld, P, max_tiles, true, nullptr, 0, true, (T*)h->eact, L.eff_pad,
                           HyGlu{d.ff_limit, d.ff_alpha, d.ff_shift, nullptr, nullptr, 0, 0, d.ff_act}, top, on_out ? nullptr : h->wsel);
    } else {
        hipLaunchKernelGGL(hy_moe_group_kernel, dim3(1), dim3(256), (size_t)2 * E * 4, st, h->sel, P, E, HY_MOE_BM, h->pair_row, h->tiles, h->ntiles);
        hipLaunchKernelGGL((hy_moe_scale_kernel<T>), dim3(P), dim3(256), 0, st, hb, W, top, on_out ? (const float*)nullptr : h->wsel, h->pair_row, (T*)h->ea);
        hy_gemm_grouped<T>(ctx, (const T*)h->ea, W, one_gu, (size_t)2 * L.eff_pad * L.egu.ld, P, max_tiles, false, nullptr, 0, true, (T*)h->eact, L.eff_pad,
                           HyGlu{d.ff_limit, d.ff_alpha, d.ff_shift, nullptr, nullptr, 0, 0, d.ff_act});
    }
    hy_gemm_grouped<T>(ctx, (const T*)h->eact, L.eff_pad, one_down, (size_t)W * L.edown.ld, P, max_tiles, few, h->eout, W, false, nullptr, 0, HyGlu{});
    if (d.shared_ff > 0) {
        T* act = (T*)h->mixo;
        hy_gemm<T>(ctx, hb, W, L.gu, n, nullptr, 0, true, act, L.ff_pad, hy_ff_glu(L));
        hy_gemm<T>(ctx, act, L.ff_pad, L.down, n, h->y, W, false, nullptr, 0, HyGlu{}, &h->y_parts);
    }
}

// logits of the nw rows listed in h->want: final norm of the gathered rows, the head's product, the optional cap * tanh(. / cap)
template <typename T>
static void hy_logits(gl3_ctx* ctx, int nw) {
    gl3_hybrid_state* h = ctx->hy;
    T* xw = (T*)h->xw;
    hy_streams<T>(ctx, nw, h->X, h->W, h->S, (size_t)h->mb * h->W, (const float*)nullptr, 1, 0, (const float*)nullptr, (const float*)nullptr,
                  h->ones, h->final_norm, ctx->d.rms_eps, xw, (float*)nullptr, h->want);
    hy_gemm<T>(ctx, xw, h->W, h->head, nw, h->logits, ctx->d.vocab, false, nullptr, 0, HyGlu{});
    if (h->softcap > 0.f) {
        const size_t cnt = (size_t)nw * ctx->d.vocab;
        hipLaunchKernelGGL(hy_softcap_kernel, dim3((unsigned)std::min<size_t>(1024, (cnt + 255) / 256)), dim3(256), 0, ctx->stream, h->logits, cnt, h->softcap);
    }
}

template <typename T>
static void hy_resid(gl3_ctx* ctx, int n, const HyResid& r, T* xt, T* h_out) {
    const bool v4 = r.W % 4 == 0;
    if (n <= 32) {
        if (v4) hipLaunchKernelGGL((hy_resid_kernel<T, 1024, 4>), dim3(n), dim3(1024), 0, ctx->stream, r, xt, h_out);
        else hipLaunchKernelGGL((hy_resid_kernel<T, 1024, 1>), dim3(n), dim3(1024), 0, ctx->stream, r, xt, h_out);
    } else {
        if (v4) hipLaunchKernelGGL((hy_resid_kernel<T, 256, 4>), dim3(n), dim3(256), 0, ctx->stream, r, xt, h_out);
        else hipLaunchKernelGGL((hy_resid_kernel<T, 256, 1>), dim3(n), dim3(256), 0, ctx->stream, r, xt, h_out);
    }
}

// One portion of a plain-residual design: x <- x + mixer(norm1 x); x <- x + ff(norm2 x); x <- x + side input; what goes on is the depth
// average.  Every residual update carries what follows it as far as the next matrix product (hy_resid_kernel).
template <typename T>
static int32_t hy_portion_plain(gl3_ctx* ctx, int seq, const int32_t* tokens, int n, int pos0, const int32_t* want, int nw) {
    gl3_hybrid_state* h = ctx->hy;
    hipStream_t st = ctx->stream;
    const int W = h->W, nl = (int)h->L.size();
    const size_t lstride = (size_t)h->mb * W;
    const float eps = ctx->d.rms_eps;
    memcpy(h->h_tokens, tokens, (size_t)n * 4);
    if (nw > 0) memcpy(h->h_want, want, (size_t)nw * 4);
    h->h_dyn[0] = pos0; h->h_dyn[1] = seq;
    HY_HIP(hipMemcpyAsync(h->dyn, h->h_dyn, (size_t)(4 + h->want_cap + n) * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL((hy_embed_kernel<T>), dim3(n, n <= 32 ? hy_cdiv(W, 256) : 1), dim3(256), 0, st, h->tokens, (const T*)h->emb.w, h->X, W, 1, lstride, h->emb_scale, h->depth ? h->hist : nullptr);
    T* hb = (T*)h->h;
    HyResid base{};
    base.x = h->X; base.W = W; base.eps = eps; base.ya_parts = 1; base.ya_mul = 1.f;
    {
        HyResid r = base;
        r.norm_w = h->L[0].norm1;
        hy_resid<T>(ctx, n, r, (T*)nullptr, hb);
    }
    for (int l = 0; l < nl; ++l) {
        HyLayer& L = h->L[l];
        const bool last = l + 1 == nl;
        // the last residual update of the layer: [side input,] depth average, tap, the next layer's norm
        auto finish = [&](HyResid r) {
            if (h->side_dim > 0) {
                hy_resid<T>(ctx, n, r, (T*)h->xb, (T*)nullptr);
                if (n <= 8) {        // gate product with gelu_tanh(.) * the token's side embedding in the epilogue -> the projection's operand
                    hy_gemm<T>(ctx, (const T*)h->xb, W, L.side_gate, n, nullptr, 0, false, (T*)h->side_g, h->side_ld,
                               HyGlu{0.f, 0.f, 0.f, h->side_emb.w, h->tokens, h->side_emb.ld, l * h->side_dim});
                } else {             // few result rows and a long K: K-split parts, added by the activation kernel
                    int sp = 1;
                    hy_gemm<T>(ctx, (const T*)h->xb, W, L.side_gate, n, h->side_z, h->side_dim, false, nullptr, 0, HyGlu{}, &sp, HY_ZSPLIT);
                    hipLaunchKernelGGL((hy_side_act_kernel<T>), dim3(n), dim3(256), 0, st, h->side_z, h->side_dim, sp, (size_t)n * h->side_dim, h->tokens,
                                       (const T*)h->side_emb.w, h->side_emb.ld, l * h->side_dim, (T*)h->side_g, h->side_ld);
                }
                hy_gemm<T>(ctx, (const T*)h->side_g, h->side_ld, L.side_proj, n, h->y, W, false, nullptr, 0, HyGlu{});
                r = base;
                r.yc = h->y; r.cw = L.side_norm;
            }
            if (h->depth) { r.hist = h->hist; r.hist_stride = lstride; r.n_mix = l + 2; r.mix = L.depth_mix; }
            if (h->taps) r.tap = h->taps + (size_t)l * lstride;
            if (!last) r.norm_w = h->L[l + 1].norm1;
            hy_resid<T>(ctx, n, r, (T*)nullptr, hb);
        };
        int32_t rc = hy_mixer<T>(ctx, L, n, pos0, seq);
        if (rc != GL3_OK) return rc;
        HyResid r = base;
        r.ya = h->y; r.ya_parts = h->y_parts; r.ya_stride = (size_t)n * W;
        if (h->parallel) {
            // one norm, two readers: the feed-forward takes the same normed rows as the mixer, its down projection's parts follow the
            // mixer's in y, and one residual update adds them all: x += residual multiplier * (mixer + feed-forward)
            if (L.d.ff > 0) {
                T* act = (T*)h->mixo;
                int p2 = 1;
                hy_gemm<T>(ctx, hb, W, L.gu, n, nullptr, 0, true, act, L.ff_pad, hy_ff_glu(L));
                hy_gemm<T>(ctx, act, L.ff_pad, L.down, n, h->y + (size_t)h->y_parts * n * W, W, false, nullptr, 0, HyGlu{}, &p2);
                r.ya_parts += p2;
            }
            r.ya_mul = h->resid_mul;
            if (h->taps) r.tap = h->taps + (size_t)l * lstride;
            if (!last) r.norm_w = h->L[l + 1].norm1;
            hy_resid<T>(ctx, n, r, (T*)nullptr, hb);
            continue;
        }
        r.post_w = L.norm1b;          // null without post norms
        if (L.d.ff > 0) {
            r.norm_w = L.norm2;
            hy_resid<T>(ctx, n, r, (T*)nullptr, hb);
            r = base;
            r.post_w = L.norm2b;
            if (L.d.experts > 0) {
                hy_moe<T>(ctx, L, n);
                r.eo = h->eout; r.pair_row = h->pair_row; r.top = L.d.top;
                if (L.d.route_on_output) r.ew = h->wsel;
                if (L.d.shared_ff > 0) {
                    r.ya = h->y; r.ya_parts = h->y_parts; r.ya_stride = (size_t)n * W;
                    if (!L.d.shared_ungated) { r.gate_z = h->sgz; r.gate_ld = 1; }
                }
            } else {
                T* act = (T*)h->mixo;
                if (L.d.ff_act == 2) hy_gemm<T>(ctx, hb, W, L.gu, n, nullptr, 0, false, act, L.ff_pad, HyGlu{0.f, 0.f, 0.f, nullptr, nullptr, 0, 0, 2});      // no gate: relu(up)^2
                else hy_gemm<T>(ctx, hb, W, L.gu, n, nullptr, 0, true, act, L.ff_pad, hy_ff_glu(L));
                hy_gemm<T>(ctx, act, L.ff_pad, L.down, n, h->y, W, false, nullptr, 0, HyGlu{}, &h->y_parts);
                r.ya = h->y; r.ya_parts = h->y_parts; r.ya_stride = (size_t)n * W;
            }
        }
        finish(r);
    }
    if (nw > 0) hy_logits<T>(ctx, nw);
    HY_HIP(hipGetLastError());
    return GL3_OK;
}

// one portion: n <= mb tokens of slot seq at pos0; wanted rows (portion-relative, nw <= want_cap) -> h->logits[nw][vocab]
template <typename T>
static int32_t hy_portion(gl3_ctx* ctx, int seq, const int32_t* tokens, int n, int pos0, const int32_t* want, int nw) {
    gl3_hybrid_state* h = ctx->hy;
    hipStream_t st = ctx->stream;
    const int W = h->W, S = h->S;
    const size_t sstride = (size_t)h->mb * W;
    const float eps = ctx->d.rms_eps;
    memcpy(h->h_tokens, tokens, (size_t)n * 4);
    if (nw > 0) memcpy(h->h_want, want, (size_t)nw * 4);
    h->h_dyn[0] = pos0; h->h_dyn[1] = seq;
    HY_HIP(hipMemcpyAsync(h->dyn, h->h_dyn, (size_t)(4 + h->want_cap + n) * 4, hipMemcpyHostToDevice, st));
    hipLaunchKernelGGL((hy_embed_kernel<T>), dim3(n, n <= 32 ? hy_cdiv(W, 256) : 1), dim3(256), 0, st, h->tokens, (const T*)h->emb.w, h->X, W, S, sstride, h->emb_scale, (float*)nullptr);
    T* hb = (T*)h->h;
    const int nl = (int)h->L.size();
    hy_streams<T>(ctx, n, h->X, W, S, sstride, (const float*)nullptr, 1, 0, (const float*)nullptr, (const float*)nullptr,
                       h->L[0].hc[0][0], h->L[0].norm1, eps, hb, (float*)nullptr, (const int*)nullptr);
    for (int l = 0; l < nl; ++l) {
        HyLayer& L = h->L[l];
        int32_t r = hy_mixer<T>(ctx, L, n, pos0, seq);
        if (r != GL3_OK) return r;
        const bool ff = L.d.ff > 0, last = l + 1 == nl;
        {   // write-back of the mixer sublayer + read of the next sublayer
            const float* nin = ff ? L.hc[1][0] : last ? nullptr : h->L[l + 1].hc[0][0];
            const float* nw_ = ff ? L.norm2 : last ? nullptr : h->L[l + 1].norm1;
            hy_streams<T>(ctx, n, h->X, W, S, sstride, h->y, h->y_parts, (size_t)n * W, L.hc[0][2], L.hc[0][1], nin, nw_, eps, hb,
                               (!ff && h->taps) ? h->taps + (size_t)l * sstride : nullptr, (const int*)nullptr);
        }
        if (ff) {
            T* act = (T*)h->mixo;
            hy_gemm<T>(ctx, hb, W, L.gu, n, nullptr, 0, true, act, L.ff_pad, hy_ff_glu(L));
            hy_gemm<T>(ctx, act, L.ff_pad, L.down, n, h->y, W, false, nullptr, 0, HyGlu{}, &h->y_parts);
            const float* nin = last ? nullptr : h->L[l + 1].hc[0][0];
            const float* nw_ = last ? nullptr : h->L[l + 1].norm1;
            hy_streams<T>(ctx, n, h->X, W, S, sstride, h->y, h->y_parts, (size_t)n * W, L.hc[1][2], L.hc[1][1], nin, nw_, eps, hb,
                               h->taps ? h->taps + (size_t)l * sstride : nullptr, (const int*)nullptr);
        }
    }
    if (nw > 0) hy_logits<T>(ctx, nw);
    HY_HIP(hipGetLastError());
    return GL3_OK;
}

int32_t gl3_hy_step(gl3_ctx* ctx, int32_t seq, const int32_t* tokens, int32_t n, int32_t start_pos, const int32_t* want, int32_t n_want, float* logits_out) {
    gl3_hybrid_state* h = ctx->hy;
    if (!ctx->finalized) GL3_FAIL(GL3_E_STATE, "gl3_finalize has not run");
    if (seq < 0 || seq >= h->n_seqs) GL3_FAIL(GL3_E_ARG, "sequence slot out of range");
    if (n < 1 || !tokens) GL3_FAIL(GL3_E_ARG, "a step needs at least one token");
    if (start_pos != 0 && start_pos != h->len[seq]) GL3_FAIL(GL3_E_STATE, "a step continues its slot (start_pos = tokens held) or restarts it (start_pos = 0)");
    if ((int64_t)start_pos + n > ctx->d.ctx) GL3_FAIL(GL3_E_ARG, "step runs past the context length");
    if (n_want < 0 || (n_want > 0 && !want)) GL3_FAIL(GL3_E_ARG, "wanted rows need want");        // logits_out == null: the rows stay on the device
    for (int i = 0; i < n; ++i)
        if (tokens[i] < 0 || tokens[i] >= ctx->d.vocab) GL3_FAIL(GL3_E_ARG, "token id out of range");
    for (int i = 0; i < n_want; ++i)
        if (want[i] < 0 || want[i] >= n || (i && want[i] <= want[i - 1])) GL3_FAIL(GL3_E_ARG, "want must be ascending indices into the step's tokens");
    HY_HIP(hipSetDevice(ctx->d.device));
    const size_t V = ctx->d.vocab;
    int wi = 0;
    for (int off = 0; off < n; off += h->mb) {
        const int pn = std::min(h->mb, n - off);
        int we = wi;
        while (we < n_want && want[we] < off + pn) ++we;
        // the portion's wanted rows in groups of want_cap: the first group rides on the portion's run, further groups only redo the head
        int done = wi;
        bool ran = false;
        do {
            const int g = std::min(h->want_cap, we - done);
            std::vector<int32_t> rel(std::max(g, 1));
            for (int i = 0; i < g; ++i) rel[i] = want[done + i] - off;
            int32_t r;
            if (!ran) {
                if (h->plain)
                    r = h->f32 ? hy_portion_plain<float>(ctx, seq, tokens + off, pn, start_pos + off, rel.data(), g)
                               : hy_portion_plain<bf16_t>(ctx, seq, tokens + off, pn, start_pos + off, rel.data(), g);
                else
                    r = h->f32 ? hy_portion<float>(ctx, seq, tokens + off, pn, start_pos + off, rel.data(), g)
                               : hy_portion<bf16_t>(ctx, seq, tokens + off, pn, start_pos + off, rel.data(), g);
                ran = true;
            } else {
                memcpy(h->h_want, rel.data(), (size_t)g * 4);
                HY_HIP(hipMemcpyAsync(h->want, h->h_want, (size_t)g * 4, hipMemcpyHostToDevice, ctx->stream));
                if (h->f32) hy_logits<float>(ctx, g); else hy_logits<bf16_t>(ctx, g);
                r = GL3_OK;
            }
            if (r != GL3_OK) return r;
            if (g > 0 && logits_out) HY_HIP(hipMemcpyAsync(h->h_logits, h->logits, (size_t)g * V * 4, hipMemcpyDeviceToHost, ctx->stream));
            HY_HIP(hipStreamSynchronize(ctx->stream));
            if (g > 0 && logits_out) memcpy(logits_out + (size_t)done * V, h->h_logits, (size_t)g * V * 4);
            done += g;
        } while (done < we);
        wi = we;
        h->last_n = pn;
    }
    h->len[seq] = start_pos + n;
    return GL3_OK;
}

int32_t gl3_hy_argmax(gl3_ctx* ctx, int32_t* out) {
    hipLaunchKernelGGL(argmax_kernel, dim3(AMX_WGS), dim3(256), 0, ctx->stream, ctx->hy->logits, ctx->d.vocab, ctx->argmax);
    HY_HIP(hipMemcpyAsync(ctx->h_argmax, ctx->argmax, sizeof(int), hipMemcpyDeviceToHost, ctx->stream));
    HY_HIP(hipStreamSynchronize(ctx->stream));
    *out = *ctx->h_argmax;
    return GL3_OK;
}

int32_t gl3_hy_seq_acquire(gl3_ctx* ctx, int32_t* seq_out) {
    gl3_hybrid_state* h = ctx->hy;
    for (int s = 0; s < h->n_seqs; ++s)
        if (!h->busy[s]) { h->busy[s] = 1; h->len[s] = 0; *seq_out = s; return GL3_OK; }
    GL3_FAIL(GL3_E_STATE, "no free sequence slot");
}
int32_t gl3_hy_seq_release(gl3_ctx* ctx, int32_t seq) {
    gl3_hybrid_state* h = ctx->hy;
    if (seq < 0 || seq >= h->n_seqs) GL3_FAIL(GL3_E_ARG, "sequence slot out of range");
    h->busy[seq] = 0; h->len[seq] = 0;
    return GL3_OK;
}
int32_t gl3_hy_reset(gl3_ctx* ctx) {
    gl3_hybrid_state* h = ctx->hy;
    std::fill(h->len.begin(), h->len.end(), 0);
    return GL3_OK;
}
int32_t gl3_hy_layer_rows(gl3_ctx* ctx, int32_t layer, float* out, int32_t n) {
    gl3_hybrid_state* h = ctx->hy;
    if (!h->taps) GL3_FAIL(GL3_E_STATE, "plan was created without GL3_FLAG_LAYER_TAPS");
    if (layer < 0 || layer >= (int)h->L.size() || n < 1 || n > h->last_n || !out) GL3_FAIL(GL3_E_ARG, "layer or row count out of range");
    HY_HIP(hipMemcpy(out, h->taps + (size_t)layer * h->mb * h->W, (size_t)n * h->W * 4, hipMemcpyDeviceToHost));
    return GL3_OK;
}

// ---- one GEMM class timed alone ---------------------------------------------------------------------------------------------------
int32_t gl3_hy_profile_gemm(int32_t device, int32_t f32, int32_t rows, int32_t k, int32_t m, int32_t glu, int32_t iters, double* out_us) {
    if (rows < 2 || k < 1 || m < 1 || iters < 1 || !out_us || (glu == 1 && rows % 64) || glu < 0 || glu > 2) return GL3_E_ARG;
    if (hipSetDevice(device) != hipSuccess) return GL3_E_HIP;
    gl3_ctx tmp; gl3_hybrid_state hs; tmp.hy = &hs; hs.f32 = f32 != 0;
    gl3_ctx* ctx = &tmp;
    const size_t es = f32 ? 4 : 2;
    // several copies of the matrix, used in rotation, so that no launch finds its weights in a cache
    const int copies = (int)std::max<size_t>(2, std::min<size_t>(16, ((size_t)1 << 30) / ((size_t)rows * k * es) + 1));
    void *w = nullptr, *a = nullptr, *act = nullptr; float* c = nullptr;
    int32_t rc = GL3_E_HIP;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    if (hipStreamCreateWithFlags(&tmp.stream, hipStreamNonBlocking) != hipSuccess) { tmp.hy = nullptr; return GL3_E_HIP; }
    do {
        if (hipMalloc(&w, (size_t)copies * rows * k * es + GL3_TAIL_PAD) != hipSuccess) { rc = GL3_E_OOM; break; }
        if (hipMalloc(&a, (size_t)m * k * es + GL3_TAIL_PAD) != hipSuccess) { rc = GL3_E_OOM; break; }
        if (hipMalloc((void**)&c, (size_t)HY_KSPLIT * m * rows * 4) != hipSuccess) { rc = GL3_E_OOM; break; }
        if (hipMalloc(&act, (size_t)m * rows * es) != hipSuccess) { rc = GL3_E_OOM; break; }
        hipMemset(w, 0, (size_t)copies * rows * k * es); hipMemset(a, 0, (size_t)m * k * es);
        hipEventCreate(&e0); hipEventCreate(&e1);
        auto run = [&](int it) {
            HyMat mt; mt.rows = rows; mt.k = k; mt.ld = k; mt.w = (uint8_t*)w + (size_t)(it % copies) * rows * k * es;
            int parts = 1;
            if (f32) hy_gemm<float>(ctx, (const float*)a, k, mt, m, c, rows, glu == 1, (float*)act, rows / 2, HyGlu{0.f, 1.f, 0.f}, glu == 2 ? &parts : nullptr);
            else hy_gemm<bf16_t>(ctx, (const bf16_t*)a, k, mt, m, c, rows, glu == 1, (bf16_t*)act, rows / 2, HyGlu{0.f, 1.f, 0.f}, glu == 2 ? &parts : nullptr);
        };
        for (int i = 0; i < 3; ++i) run(i);
        hipEventRecord(e0, tmp.stream);
        for (int i = 0; i < iters; ++i) run(i);
        hipEventRecord(e1, tmp.stream);
        if (hipStreamSynchronize(tmp.stream) != hipSuccess) break;
        float ms = 0.f;
        hipEventElapsedTime(&ms, e0, e1);
        *out_us = (double)ms * 1e3 / iters;
        rc = GL3_OK;
    } while (0);
    if (e0) hipEventDestroy(e0);
    if (e1) hipEventDestroy(e1);
    hipFree(w); hipFree(a); hipFree(c); hipFree(act);
    hipStreamDestroy(tmp.stream);
    tmp.stream = nullptr; tmp.hy = nullptr;
    return rc;
}
