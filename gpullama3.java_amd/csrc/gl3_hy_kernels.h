// gl3_hy_kernels.h — kernels of the layer-list family (GL3_ARCH_NODITAR): stream mixing + RMS norm, the bfloat16 / float32 MFMA GEMM and
// the small-batch matvec with their epilogues, the cache writers, the tiled softmax attention with key splits, the latent expansion,
// the short convolution, the state-space scan and its gated norm.  Every mechanism takes its sizes and constants as arguments.
//
// Number formats: T = bf16_t (matrices and GEMM inputs in bfloat16, float32 accumulation) or float (everything float32; the MFMA is
// v_mfma_f32_32x32x2_f32, a true float32 product).  Residual streams, projections' outputs, scores, softmax, norms, the convolution and
// the recurrence are float32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;

__device__ __forceinline__ float hy_bf2f(bf16_t v) { return __uint_as_float((uint32_t)v << 16); }
__device__ __forceinline__ bf16_t hy_f2bf(float f) {          // round to nearest even
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float hy_ld(const float* p) { return *p; }
__device__ __forceinline__ float hy_ld(const bf16_t* p) { return hy_bf2f(*p); }
__device__ __forceinline__ void hy_st(float* p, float v) { *p = v; }
__device__ __forceinline__ void hy_st(bf16_t* p, float v) { *p = hy_f2bf(v); }

__device__ __forceinline__ float hy_sigmoid(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float hy_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float hy_softplus(float z) { return z > 20.f ? z : log1pf(expf(z)); }

__device__ __forceinline__ float hy_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float hy_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// sum over the NT threads of a workgroup; red = float[NT / 64] in LDS; every thread gets the result
template <int NT = 256>
__device__ __forceinline__ float hy_block_sum(float v, float* red) {
    v = hy_wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < NT / 64; ++i) a += red[i];
    return a;
}

// step record in device memory (read by the kernels, so that a captured step can be replayed at another position):
// dyn[0] = position of the step's first token, dyn[1] = sequence slot
constexpr int HY_MAX_STREAMS = 8;

// ---- embedding: every stream starts as the token's row times `scale`; copy != null keeps the embedding output for the depth average --
template <typename T>
static __global__ __launch_bounds__(256) void hy_embed_kernel(const int* __restrict__ tokens, const T* __restrict__ emb, float* __restrict__ X,
                                                              int W, int S, size_t sstride, float scale, float* __restrict__ copy) {
    const int t = blockIdx.x;
    const T* row = emb + (size_t)tokens[t] * W;
    for (int w = blockIdx.y * 256 + threadIdx.x; w < W; w += 256 * gridDim.y) {
        const float v = hy_ld(row + w) * scale;
        for (int s = 0; s < S; ++s) X[s * sstride + (size_t)t * W + w] = v;
        if (copy) copy[(size_t)t * W + w] = v;
    }
}

// ---- stream tables + norm -----------------------------------------------------------------------------------------------------
// One workgroup per token.  "post" (y != null): x_t <- sum_s mix[s][t] x_s + out[t] y for all streams at once.  "pre" (pre_in != null):
// u = sum_s in[s] x_s, h = u / sqrt(mean(u^2) + eps) * norm_w, written as TO.  sum_out (taps): the plain sum of the streams.
// rows != null: workgroup b reads token rows[b] and writes row b of h_out (the gather in front of the output head).
// NT threads per token: 256 for portions with many tokens, 1024 for a few tokens (a thread's element loop is a chain of dependent
// load - store round trips).  The first HY_UR values of u per thread stay in registers for the second pass.
constexpr int HY_UR = 8;
template <typename TO, int NT>
static __global__ __launch_bounds__(NT) void hy_streams_kernel(float* __restrict__ X, int W, int S, size_t sstride, const float* __restrict__ y, int yparts, size_t ystride,
                                                                const float* __restrict__ post_mix, const float* __restrict__ post_out,
                                                                const float* __restrict__ pre_in, const float* __restrict__ norm_w, float eps,
                                                                TO* __restrict__ h_out, float* __restrict__ sum_out, const int* __restrict__ rows) {
    __shared__ float red[NT / 64];
    const int b = blockIdx.x, t = rows ? rows[b] : b;
    float mix[HY_MAX_STREAMS * HY_MAX_STREAMS], po[HY_MAX_STREAMS], pi[HY_MAX_STREAMS], ur[HY_UR];
#pragma unroll
    for (int s = 0; s < HY_MAX_STREAMS; ++s) {
        po[s] = (y && s < S) ? post_out[s] : 0.f;
        pi[s] = (pre_in && s < S) ? pre_in[s] : 0.f;
#pragma unroll
        for (int u = 0; u < HY_MAX_STREAMS; ++u) mix[s * HY_MAX_STREAMS + u] = (y && s < S && u < S) ? post_mix[s * S + u] : 0.f;
    }
    float ss = 0.f;
    int it = 0;
    for (int w = threadIdx.x; w < W; w += NT, ++it) {
        float xs[HY_MAX_STREAMS];
#pragma unroll
        for (int s = 0; s < HY_MAX_STREAMS; ++s) xs[s] = s < S ? X[s * sstride + (size_t)t * W + w] : 0.f;
        if (y) {
            float yv = y[(size_t)t * W + w];                         // the sublayer's output may come as K-split partial sums
            for (int z = 1; z < yparts; ++z) yv += y[z * ystride + (size_t)t * W + w];
            float nx[HY_MAX_STREAMS];
#pragma unroll
            for (int u = 0; u < HY_MAX_STREAMS; ++u) {
                float a = 0.f;
#pragma unroll
                for (int s = 0; s < HY_MAX_STREAMS; ++s) a += mix[s * HY_MAX_STREAMS + u] * xs[s];
                nx[u] = a + po[u] * yv;
            }
#pragma unroll
            for (int s = 0; s < HY_MAX_STREAMS; ++s) {
                xs[s] = nx[s];
                if (s < S) X[s * sstride + (size_t)t * W + w] = nx[s];
            }
        }
        if (sum_out) {
            float a = 0.f;
#pragma unroll
            for (int s = 0; s < HY_MAX_STREAMS; ++s) a += xs[s];
            sum_out[(size_t)b * W + w] = a;
        }
        if (pre_in) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < HY_MAX_STREAMS; ++s) u += pi[s] * xs[s];
            ss += u * u;
#pragma unroll
            for (int q = 0; q < HY_UR; ++q)
                if (q == it) ur[q] = u;
        }
    }
    if (!pre_in) return;
    ss = hy_block_sum<NT>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)W + eps);
#pragma unroll
    for (int q = 0; q < HY_UR; ++q) {
        const int w = threadIdx.x + q * NT;
        if (w < W) hy_st(h_out + (size_t)b * W + w, ur[q] * r * norm_w[w]);
    }
    // wider rows: a thread re-reads what it wrote above (same w, same sum)
    for (int w = threadIdx.x + HY_UR * NT; w < W; w += NT) {
        float u = 0.f;
#pragma unroll
        for (int s = 0; s < HY_MAX_STREAMS; ++s) u += pi[s] * (s < S ? X[s * sstride + (size_t)t * W + w] : 0.f);
        hy_st(h_out + (size_t)b * W + w, u * r * norm_w[w]);
    }
}

// ---- GEMM: C[m][n] = sum_k A[m][k] W[n][k]  (tokens x features, both operands K-contiguous) --------------------------------------
typedef float hy_v16f __attribute__((ext_vector_type(16)));

// Epilogues: STORE = the float32 products; GLU = gate / up pairs -> activation in the matrix type; ACTMUL = act(product) in the matrix
// type: gelu_tanh(product) times an entry of a per-token table row (mul_table[mul_rows[m]][mul_col0 + feature], the per-layer token
// input), or relu(product)^2 alone (act = 2, mul_table = null: a feed-forward without a gate).
enum { HY_EPI_STORE = 0, HY_EPI_GLU = 1, HY_EPI_ACTMUL = 2 };
struct HyGlu { float limit, alpha, shift; const void* mul_table; const int* mul_rows; int mul_ld, mul_col0; int act; };      // act 1: gelu_tanh(g) u; 2: relu(u)^2, no gate
__device__ __forceinline__ float hy_gelu_tanh(float z) { return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }
template <typename T>
__device__ __forceinline__ float hy_actmul(float a, int m, int feature, const HyGlu& p) {
    if (p.act == 2) { const float r = fmaxf(a, 0.f); return r * r; }
    return hy_gelu_tanh(a) * hy_ld((const T*)p.mul_table + (size_t)p.mul_rows[m] * p.mul_ld + p.mul_col0 + feature);
}
__device__ __forceinline__ float hy_glu(float g, float u, const HyGlu& p) {
    if (p.limit > 0.f) { g = fminf(g, p.limit); u = fminf(fmaxf(u, -p.limit), p.limit); }
    if (p.act == 1) return hy_gelu_tanh(g) * u;
    return g * hy_sigmoid(p.alpha * g) * (u + p.shift);
}

template <typename T> struct HyPiece;          // 16 bytes of an operand row
// N elements per piece, PPR pieces per tile row and K step (K step = N PPR elements), LDS row stride in elements (K step + pad)
template <> struct HyPiece<bf16_t> { static constexpr int N = 8; static constexpr int PPR = 8; static constexpr int LDS_STRIDE = 72; };
template <> struct HyPiece<float> { static constexpr int N = 4; static constexpr int PPR = 4; static constexpr int LDS_STRIDE = 17; };
typedef __bf16 hy_v8bf __attribute__((ext_vector_type(8)));

template <typename T>
__device__ __forceinline__ uint4 hy_load_piece(const T* __restrict__ base, int ld, int row, int rows, int k, int K, bool vec_ok) {
    constexpr int PE = HyPiece<T>::N;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (row >= rows || k >= K) return v;
    const T* p = base + (size_t)row * ld + k;
    if (vec_ok && k + PE <= K) return *reinterpret_cast<const uint4*>(p);
    __attribute__((aligned(16))) T tmp[PE];
#pragma unroll
    for (int i = 0; i < PE; ++i) tmp[i] = (k + i < K) ? p[i] : (T)0;
    return *reinterpret_cast<uint4*>(tmp);
}

// Workgroup = 4 wavefronts in 2 x 2, tile BM tokens x BN features, K step = 64 bfloat16 (v_mfma_f32_32x32x16_bf16) / 16 float32
// (v_mfma_f32_32x32x2_f32); the next K step's pieces travel in registers under the current step's MFMAs.  EPI_GLU: W's rows come in blocks of 64 = 32 gate rows followed by the 32
// up rows of the same features, so one lane holds gate and up of a (token, feature) and writes the activation act[m][feature].
// Grouped form (GR = 1, mixture of experts): blockIdx.y walks a list of row tiles {first row, rows (<= BM), expert} that a device kernel
// made (hy_moe_group_kernel); the tile's rows of A / C / act are consecutive, its weights are the expert's N rows of the stacked matrix
// (wstride elements per expert).  Workgroups past the list's length leave at once.
struct HyGroup { const int* tiles; const int* ntiles; size_t wstride; };
template <typename T, typename TO, int BM, int BN, int EPI, int GR = 0>
static __global__ __launch_bounds__(256) void hy_gemm_kernel(const T* __restrict__ A, int lda, const T* __restrict__ Wt, int ldw, int M, int N, int K,
                                                             float* __restrict__ C, int ldc, TO* __restrict__ act, int ld_act, HyGlu glu, int kper, HyGroup grp = HyGroup{}) {
    int m0 = blockIdx.y * BM;
    if constexpr (GR) {
        if ((int)blockIdx.y >= grp.ntiles[0]) return;
        const int* tl = grp.tiles + 3 * blockIdx.y;
        const int row0 = tl[0];
        M = tl[1];
        A += (size_t)row0 * lda;
        Wt += (size_t)tl[2] * grp.wstride;
        if (C) C += (size_t)row0 * ldc;
        if (act) act += (size_t)row0 * ld_act;
        m0 = 0;
    }
    // blockIdx.z = K split: this launch's workgroup sums k in [z kper, (z + 1) kper) into its own copy of C (STORE only; kper is a multiple of the K step)
    const int kbeg = blockIdx.z * kper, kend = min(K, kbeg + kper);
    C += (size_t)blockIdx.z * M * ldc;
    constexpr int PE = HyPiece<T>::N, PPR = HyPiece<T>::PPR, BK = PPR * PE, LS = HyPiece<T>::LDS_STRIDE;
    constexpr int TM = BM / 64, TN = BN / 64, PA = BM * PPR / 256, PW = BN * PPR / 256;
    __shared__ __attribute__((aligned(16))) T sA[BM * LS];
    __shared__ __attribute__((aligned(16))) T sW[BN * LS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int n0 = blockIdx.x * BN;
    const bool va = (lda % PE) == 0 && ((uintptr_t)A % 16) == 0, vw = (ldw % PE) == 0 && ((uintptr_t)Wt % 16) == 0;
    hy_v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    uint4 ra[PA], rw[PW];
    auto gload = [&](int k0) {
#pragma unroll
        for (int i = 0; i < PA; ++i) { const int id = tid + i * 256; ra[i] = hy_load_piece<T>(A, lda, m0 + id / PPR, M, k0 + (id % PPR) * PE, kend, va); }
#pragma unroll
        for (int i = 0; i < PW; ++i) { const int id = tid + i * 256; rw[i] = hy_load_piece<T>(Wt, ldw, n0 + id / PPR, N, k0 + (id % PPR) * PE, kend, vw); }
    };
    auto sstore = [&]() {
#pragma unroll
        for (int i = 0; i < PA; ++i) {
            const int id = tid + i * 256;
            if constexpr (sizeof(T) == 2) *reinterpret_cast<uint4*>(sA + (id / PPR) * LS + (id % PPR) * PE) = ra[i];       // 144-byte rows: 16-byte aligned
            else { uint32_t* d = reinterpret_cast<uint32_t*>(sA + (id / PPR) * LS + (id % PPR) * PE); d[0] = ra[i].x; d[1] = ra[i].y; d[2] = ra[i].z; d[3] = ra[i].w; }
        }
#pragma unroll
        for (int i = 0; i < PW; ++i) {
            const int id = tid + i * 256;
            if constexpr (sizeof(T) == 2) *reinterpret_cast<uint4*>(sW + (id / PPR) * LS + (id % PPR) * PE) = rw[i];
            else { uint32_t* d = reinterpret_cast<uint32_t*>(sW + (id / PPR) * LS + (id % PPR) * PE); d[0] = rw[i].x; d[1] = rw[i].y; d[2] = rw[i].z; d[3] = rw[i].w; }
        }
    };
    gload(kbeg);
    sstore();
    __syncthreads();
    for (int k0 = kbeg; k0 < kend; k0 += BK) {
        const bool more = k0 + BK < kend;
        if (more) gload(k0 + BK);
        const int r32 = lane & 31, kh = lane >> 5;
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 16) {          // lane: row lane % 32, k = kk + 8 (lane / 32) .. + 8
                hy_v8bf fa[TM], fw[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const hy_v8bf*>(sA + (wm * (BM / 2) + i * 32 + r32) * LS + kk + 8 * kh);
#pragma unroll
                for (int j = 0; j < TN; ++j) fw[j] = *reinterpret_cast<const hy_v8bf*>(sW + (wn * (BN / 2) + j * 32 + r32) * LS + kk + 8 * kh);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
            }
        } else {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 2) {
                float fa[TM], fw[TN];
#pragma unroll
                for (int i = 0; i < TM; ++i) fa[i] = *reinterpret_cast<const float*>(sA + (wm * (BM / 2) + i * 32 + r32) * LS + kk + kh);
#pragma unroll
                for (int j = 0; j < TN; ++j) fw[j] = *reinterpret_cast<const float*>(sW + (wn * (BN / 2) + j * 32 + r32) * LS + kk + kh);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fw[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
        if (more) { sstore(); __syncthreads(); }
    }
    // lane holds column lane % 32 and rows 8 (r / 4) + 4 (lane / 32) + r % 4 of every 32 x 32 tile
    const int col = lane & 31, rbase = 4 * (lane >> 5);
    if constexpr (EPI == HY_EPI_STORE || EPI == HY_EPI_ACTMUL) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = n0 + wn * (BN / 2) + j * 32 + col;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + rbase + (r & 3);
                    if (m < M && n < N) {
                        if constexpr (EPI == HY_EPI_STORE) C[(size_t)m * ldc + n] = acc[i][j][r];
                        else hy_st(act + (size_t)m * ld_act + n, hy_actmul<T>(acc[i][j][r], m, n, glu));
                    }
                }
            }
    } else {
        static_assert(EPI != HY_EPI_GLU || TN % 2 == 0, "gate / up pairs need a wavefront tile of 64 features");
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; j += 2) {
                const int f = (n0 + wn * (BN / 2) + j * 32) / 2 + col;        // feature of this lane's gate (tile j) and up (tile j + 1)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int m = m0 + wm * (BM / 2) + i * 32 + 8 * (r >> 2) + rbase + (r & 3);
                    if (m < M && f < ld_act && 2 * f < N) hy_st(act + (size_t)m * ld_act + f, hy_glu(acc[i][j][r], acc[i][j + 1][r], glu));
                }
            }
    }
}

// Small batches (decode): a pair of weight rows x MT tokens; the weights are read once, 16 bytes per lane and step.  KS = 1: one
// wavefront per pair (4 pairs per workgroup); KS = 4: the workgroup's four wavefronts split K of ONE pair and meet in LDS — four times
// the wavefronts in flight for matrices with few rows.  EPI_GLU: the pair is (gate row, up row) of one feature in the block layout above.
// Grouped form (GR = 1, mixture of experts, MT = 1): blockIdx.y = a (token, choice) pair whose expert sel[pair] picks the N rows of the
// stacked matrix; row `pair` of A, C and act belongs to it.
template <typename T, typename TO, int MT, int EPI, int KS, int GR = 0>
static __global__ __launch_bounds__(256) void hy_matvec_kernel(const T* __restrict__ A, int lda, const T* __restrict__ Wt, int ldw, int M, int N, int K,
                                                               float* __restrict__ C, int ldc, TO* __restrict__ act, int ld_act, HyGlu glu,
                                                               const int* __restrict__ sel = nullptr, size_t wstride = 0, int a_div = 1,
                                                               const float* __restrict__ row_scale = nullptr) {
    constexpr int PE = HyPiece<T>::N;
    float rs = 1.f;          // grouped: the pair's products are multiplied by row_scale[pair] (a score that scales the expert's input scales W x)
    if constexpr (GR) {
        const int pair_ = blockIdx.y;
        A += (size_t)(pair_ / a_div) * lda;          // a_div = choices per token: the pairs of a token share its row
        if (row_scale) rs = row_scale[pair_];
        Wt += (size_t)sel[pair_] * wstride;
        if (C) C += (size_t)pair_ * ldc;
        if (act) act += (size_t)pair_ * ld_act;
    }
    __shared__ float red[3][2 * MT];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int pair = KS == 1 ? blockIdx.x * 4 + wave : blockIdx.x;
    const int kt = KS == 1 ? lane : threadIdx.x, kstep = KS == 1 ? 64 : 256;          // this thread's place in the walk over K
    int r0, r1;
    if constexpr (EPI == HY_EPI_GLU) { r0 = (pair >> 5) * 64 + (pair & 31); r1 = r0 + 32; }
    else { r0 = 2 * pair; r1 = r0 + 1; }
    if (r0 >= N) return;                                                               // uniform per workgroup when KS = 4
    const bool has1 = r1 < N;
    const T* w0 = Wt + (size_t)r0 * ldw;
    const T* w1 = Wt + (size_t)(has1 ? r1 : r0) * ldw;
    float a0[MT], a1[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) a0[m] = a1[m] = 0.f;
    const bool vec = (lda % PE) == 0 && (ldw % PE) == 0 && ((uintptr_t)A % 16) == 0 && ((uintptr_t)Wt % 16) == 0;
    const int kv = vec ? (K / PE) * PE : 0;
#pragma unroll 2
    for (int k = kt * PE; k < kv; k += kstep * PE) {
        const uint4 p0 = *reinterpret_cast<const uint4*>(w0 + k), p1 = *reinterpret_cast<const uint4*>(w1 + k);
        float f0[PE], f1[PE];
        if constexpr (sizeof(T) == 2) {
            const uint32_t u0[4] = {p0.x, p0.y, p0.z, p0.w}, u1[4] = {p1.x, p1.y, p1.z, p1.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f0[2 * i] = __uint_as_float(u0[i] << 16); f0[2 * i + 1] = __uint_as_float(u0[i] & 0xffff0000u);
                f1[2 * i] = __uint_as_float(u1[i] << 16); f1[2 * i + 1] = __uint_as_float(u1[i] & 0xffff0000u);
            }
        } else {
            f0[0] = __uint_as_float(p0.x); f0[1] = __uint_as_float(p0.y); f0[2] = __uint_as_float(p0.z); f0[3] = __uint_as_float(p0.w);
            f1[0] = __uint_as_float(p1.x); f1[1] = __uint_as_float(p1.y); f1[2] = __uint_as_float(p1.z); f1[3] = __uint_as_float(p1.w);
        }
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m < M) {
                const uint4 pa = *reinterpret_cast<const uint4*>(A + (size_t)m * lda + k);
                float fa[PE];
                if constexpr (sizeof(T) == 2) {
                    const uint32_t ua[4] = {pa.x, pa.y, pa.z, pa.w};
#pragma unroll
                    for (int i = 0; i < 4; ++i) { fa[2 * i] = __uint_as_float(ua[i] << 16); fa[2 * i + 1] = __uint_as_float(ua[i] & 0xffff0000u); }
                } else {
                    fa[0] = __uint_as_float(pa.x); fa[1] = __uint_as_float(pa.y); fa[2] = __uint_as_float(pa.z); fa[3] = __uint_as_float(pa.w);
                }
#pragma unroll
                for (int i = 0; i < PE; ++i) { a0[m] = fmaf(fa[i], f0[i], a0[m]); a1[m] = fmaf(fa[i], f1[i], a1[m]); }
            }
        }
    }
    for (int k = kv + kt; k < K; k += kstep) {
        const float x0 = hy_ld(w0 + k), x1 = hy_ld(w1 + k);
#pragma unroll
        for (int m = 0; m < MT; ++m)
            if (m < M) { const float a = hy_ld(A + (size_t)m * lda + k); a0[m] = fmaf(a, x0, a0[m]); a1[m] = fmaf(a, x1, a1[m]); }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) { a0[m] = hy_wave_sum(a0[m]); a1[m] = hy_wave_sum(a1[m]); }
    if constexpr (KS == 4) {
        if (wave > 0 && lane == 0) {
#pragma unroll
            for (int m = 0; m < MT; ++m) { red[wave - 1][2 * m] = a0[m]; red[wave - 1][2 * m + 1] = a1[m]; }
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            a0[m] = (a0[m] + red[0][2 * m]) + (red[1][2 * m] + red[2][2 * m]);
            a1[m] = (a1[m] + red[0][2 * m + 1]) + (red[1][2 * m + 1] + red[2][2 * m + 1]);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            if (m >= M) break;
            if constexpr (EPI == HY_EPI_GLU) {
                const int f = (pair >> 5) * 32 + (pair & 31);
                if (f < ld_act) hy_st(act + (size_t)m * ld_act + f, hy_glu(a0[m] * rs, has1 ? a1[m] * rs : 0.f, glu));
            } else if constexpr (EPI == HY_EPI_ACTMUL) {
                hy_st(act + (size_t)m * ld_act + r0, hy_actmul<T>(a0[m], m, r0, glu));
                if (has1) hy_st(act + (size_t)m * ld_act + r1, hy_actmul<T>(a1[m], m, r1, glu));
            } else {
                C[(size_t)m * ldc + r0] = a0[m];
                if (has1) C[(size_t)m * ldc + r1] = a1[m];
            }
        }
    }
}

// ---- attention: cache writers ---------------------------------------------------------------------------------------------------
// One wavefront per (token, head): query heads are normalised (unit root mean square, optional) and turned by their position (optional)
// in place, key heads likewise on their way to the key rows of the slot, value heads are normalised (optional), turned (optional) and
// written to the value rows.  proj row = [.. q (H x D) .. k (G x D) .. v (G x V) ..].
// Rotary turn: entry i of the first `dims` pairs with entry i + dims / 2 (interleaved: entry 2 i with entry 2 i + 1) and the pair (u, v)
// becomes (u cos a - v sin a, v cos a + u sin a), a = pos * freq[i] in float32; freq is a table the host made (base^(-2 i / dims),
// divided for q / k by the position scaling).  An entry is (src + bias) * r * weight before it turns (bias, weight: null = absent).
struct HyRot {
    int qk_dims; const float* qk_freq;       // q / k: first qk_dims entries turn; 0 = none
    int v_norm;                              // values: unit root mean square per head
    const float* v_freq;                     // values: all V entries turn (null = none)
    int interleaved;                         // q / k pairs are (2 i, 2 i + 1)
};
// further inputs of the cache writers (null = absent): a bias per projection row, added first; weights of the norm over a whole
// projection (unit_norm = 2)
struct HyPrepX { const float* bias; const float* qn; const float* kn; const float* rowr; };
__device__ __forceinline__ void hy_turn_store(float* __restrict__ dst, const float* __restrict__ src, int D, int dims, const float* __restrict__ freq, float pos, float r, int lane,
                                              int interleaved = 0, const float* __restrict__ bias = nullptr, const float* __restrict__ w = nullptr) {
    const int half = dims >> 1;
    auto val = [&](int d) { return (src[d] + (bias ? bias[d] : 0.f)) * r * (w ? w[d] : 1.f); };
    for (int d = lane; d < half; d += 64) {
        float sn, cs;
        sincosf(pos * freq[d], &sn, &cs);
        const int i0 = interleaved ? 2 * d : d, i1 = interleaved ? 2 * d + 1 : d + half;
        const float u = val(i0), v = val(i1);
        dst[i0] = u * cs - v * sn;
        dst[i1] = v * cs + u * sn;
    }
    for (int d = dims + lane; d < D; d += 64) dst[d] = val(d);
}
static __global__ __launch_bounds__(64) void hy_attn_prep_kernel(float* __restrict__ proj, int ld, int q_off, int k_off, int v_off, int H, int G, int D, int V,
                                                                 int unit_norm, float eps, float* __restrict__ kc, float* __restrict__ vc, size_t slot_stride,
                                                                 const int* __restrict__ dyn, HyRot rot, HyPrepX x = HyPrepX{}) {
    const int t = blockIdx.x, hh = blockIdx.y, lane = threadIdx.x;
    const int pos = dyn[0] + t;
    const size_t slot = (size_t)dyn[1] * slot_stride;
    if (hh < H + G) {
        const bool isq = hh < H;
        const int col = isq ? q_off + hh * D : k_off + (hh - H) * D;
        float* src = proj + (size_t)t * ld + col;
        const float* bias = x.bias ? x.bias + col : nullptr;
        const float* w = nullptr;
        float r = 1.f;
        if (unit_norm == 2) {          // over the whole projection: hy_rowrms_kernel has left 1 / rms of the token's q and k rows
            r = x.rowr[2 * t + (isq ? 0 : 1)];
            w = (isq ? x.qn : x.kn) + (isq ? hh : hh - H) * D;
        } else if (unit_norm) {
            float ss = 0.f;
            for (int d = lane; d < D; d += 64) { const float v = src[d] + (bias ? bias[d] : 0.f); ss += v * v; }
            ss = hy_wave_sum(ss);
            r = 1.f / sqrtf(ss / (float)D + eps);
        }
        float* dst = isq ? src : kc + slot + (size_t)pos * (G * D) + (hh - H) * D;
        if (isq && !unit_norm && !rot.qk_dims && !bias) return;
        hy_turn_store(dst, src, D, rot.qk_dims, rot.qk_freq, (float)pos, r, lane, rot.interleaved, bias, w);      // a lane reads both entries of its pairs before it writes them
    } else {
        const int g = hh - H - G;
        const float* src = proj + (size_t)t * ld + v_off + g * V;
        const float* bias = x.bias ? x.bias + v_off + g * V : nullptr;
        float* dst = vc + slot + (size_t)pos * (G * V) + g * V;
        float r = 1.f;
        if (rot.v_norm) {
            float ss = 0.f;
            for (int d = lane; d < V; d += 64) { const float v = src[d] + (bias ? bias[d] : 0.f); ss += v * v; }
            ss = hy_wave_sum(ss);
            r = 1.f / sqrtf(ss / (float)V + eps);
        }
        hy_turn_store(dst, src, V, rot.v_freq ? V : 0, rot.v_freq, (float)pos, r, lane, 0, bias);
    }
}

// 1 / sqrt(mean((x + bias)^2) + eps) over two column ranges of every token's projection row (the whole q projection and the whole k
// projection): out[2 t], out[2 t + 1].  Runs before the cache writers rewrite q in place.
template <int NT>
static __global__ __launch_bounds__(NT) void hy_rowrms_kernel(const float* __restrict__ proj, int ld, int off0, int len0, int off1, int len1,
                                                              const float* __restrict__ bias, float eps, float* __restrict__ out) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x, which = blockIdx.y, off = which ? off1 : off0, len = which ? len1 : len0;
    const float* row = proj + (size_t)t * ld + off;
    float ss = 0.f;
    for (int d0 = threadIdx.x; d0 < len; d0 += 4 * NT) {          // four loads (and their biases) in flight per thread
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) { const int d = d0 + u * NT; v[u] = d < len ? row[d] + (bias ? bias[off + d] : 0.f) : 0.f; }
#pragma unroll
        for (int u = 0; u < 4; ++u) ss += v[u] * v[u];
    }
    ss = hy_block_sum<NT>(ss, red);
    if (threadIdx.x == 0) out[2 * t + which] = 1.f / sqrtf(ss / (float)len + eps);
}

// Pooled rows of a cache: the P cached rows of run b (positions b P .. b P + P - 1) are averaged into pooled row b (summed in position
// order).  One workgroup per block that the step completes (its last position lies in the step) and cache
// (blockIdx.y = 0 keys, 1 values).
static __global__ __launch_bounds__(256) void hy_pool_kernel(const float* __restrict__ kc, const float* __restrict__ vc, float* __restrict__ pk, float* __restrict__ pv,
                                                             int ldk, int ldv, int P, size_t slot_stride, const int* __restrict__ dyn, int n) {
    const int b = dyn[0] / P + blockIdx.x;
    if ((b + 1) * P > dyn[0] + n) return;
    const size_t slot = (size_t)dyn[1] * slot_stride;
    const int ld = blockIdx.y ? ldv : ldk;
    const float* src = (blockIdx.y ? vc : kc) + slot + (size_t)b * P * ld;
    float* dst = (blockIdx.y ? pv : pk) + slot + (size_t)b * ld;
    for (int c = blockIdx.z * 256 + threadIdx.x; c < ld; c += 256 * gridDim.z) {
        float a = 0.f;
        int j = 0;
        for (; j + 8 <= P; j += 8) {          // eight rows in flight, added in position order
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(j + u) * ld + c];
#pragma unroll
            for (int u = 0; u < 8; ++u) a += v[u];
        }
        for (; j < P; ++j) a += src[(size_t)j * ld + c];
        dst[c] = a / (float)P;
    }
}

// Latent attention: the latent of every token, RMS-normed with its weight, goes to the slot's latent rows.
static __global__ __launch_bounds__(64) void hy_latent_norm_kernel(const float* __restrict__ proj, int ld, int c_off, int R, const float* __restrict__ cnorm, float eps,
                                                                   float* __restrict__ cc, size_t slot_stride, const int* __restrict__ dyn) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* src = proj + (size_t)t * ld + c_off;
    float ss = 0.f;
    for (int r = lane; r < R; r += 64) ss += src[r] * src[r];
    ss = hy_wave_sum(ss);
    const float s = 1.f / sqrtf(ss / (float)R + eps);
    float* dst = cc + (size_t)dyn[1] * slot_stride + (size_t)(dyn[0] + t) * R;
    for (int r = lane; r < R; r += 64) dst[r] = src[r] * s * cnorm[r];
}

// Latent attention with a rotated part (D unrotated + P rotated entries per query head, one rotated key part of P entries for all heads,
// cached behind the latent).  blockIdx.y = 0: the first R entries of the token's down projection are RMS-normed with their weight into
// the slot row's [0, R), the P entries behind them turn by the position into [R, R + P) (nothing when cc == null: a layer that reads
// another layer's cache).  blockIdx.y = 1 + h: the last P entries of query head h turn in place.  Turn: pair (i, i + P / 2) becomes
// (u c - v s, v c + u s), c = mscale cos(pos freq[i]), s = mscale sin(pos freq[i]).  The angle is formed and brought into (-pi, pi] in double
// (a float holds an angle of a thousand radians to 1e-4 only), sine and cosine are float32.
__device__ __forceinline__ void hy_sincos_pos(int pos, double freq, float mscale, float* sn, float* cs) {
    const double a = (double)pos * freq;
    const float r = (float)(a - 6.283185307179586476925 * rint(a * 0.15915494309189533577));
    sincosf(r, sn, cs);
    *sn *= mscale; *cs *= mscale;
}
static __global__ __launch_bounds__(64) void hy_latent_prep_kernel(float* __restrict__ q, int ldq, int D, int P, const float* __restrict__ proj, int ld, int c_off, int R,
                                                                   const float* __restrict__ cnorm, float eps, float* __restrict__ cc, size_t slot_stride,
                                                                   const int* __restrict__ dyn, const double* __restrict__ freq, float mscale) {
    const int t = blockIdx.x, lane = threadIdx.x, half = P >> 1;
    const int pos = dyn[0] + t;
    if (blockIdx.y == 0) {
        if (!cc) return;
        const float* src = proj + (size_t)t * ld + c_off;
        float ss = 0.f;
        for (int r = lane; r < R; r += 64) ss += src[r] * src[r];
        ss = hy_wave_sum(ss);
        const float s = 1.f / sqrtf(ss / (float)R + eps);
        float* dst = cc + (size_t)dyn[1] * slot_stride + (size_t)(dyn[0] + t) * (R + P);
        for (int r = lane; r < R; r += 64) dst[r] = src[r] * s * cnorm[r];
        for (int i = lane; i < half; i += 64) {
            float sn, cs;
            hy_sincos_pos(pos, freq[i], mscale, &sn, &cs);
            const float u = src[R + i], v = src[R + half + i];
            dst[R + i] = u * cs - v * sn;
            dst[R + half + i] = v * cs + u * sn;
        }
    } else {
        float* qr = q + (size_t)t * ldq + (size_t)(blockIdx.y - 1) * (D + P) + D;
        for (int i = lane; i < half; i += 64) {
            float sn, cs;
            hy_sincos_pos(pos, freq[i], mscale, &sn, &cs);
            const float u = qr[i], v = qr[half + i];
            qr[i] = u * cs - v * sn;
            qr[half + i] = v * cs + u * sn;
        }
    }
}

// out[t][0 .. len) = rms_norm(src[t][off .. off + len)) * w in the matrix type (the operand of a following product); one workgroup per token
template <typename TO>
static __global__ __launch_bounds__(256) void hy_rownorm_kernel(const float* __restrict__ src, int ld, int off, int len, const float* __restrict__ w, float eps,
                                                                TO* __restrict__ out, int ldo) {
    __shared__ float red[4];
    const int t = blockIdx.x;
    const float* row = src + (size_t)t * ld + off;
    float ss = 0.f;
    for (int i = threadIdx.x; i < len; i += 256) ss += row[i] * row[i];
    ss = hy_block_sum<256>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)len + eps);
    for (int i = threadIdx.x; i < len; i += 256) hy_st(out + (size_t)t * ldo + i, row[i] * r * w[i]);
}

// c[i] += c[stride + i] + .. + c[(parts - 1) stride + i]: the K-split parts of a product whose consumers read single entries
static __global__ __launch_bounds__(256) void hy_sum_parts_kernel(float* __restrict__ c, int parts, size_t stride, size_t n) {
    for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 4; i < n; i += (size_t)gridDim.x * 1024) {
        if (i + 4 <= n && (stride & 3) == 0) {
            float4 a = *reinterpret_cast<const float4*>(c + i);
            for (int z = 1; z < parts; ++z) { const float4 q = *reinterpret_cast<const float4*>(c + z * stride + i); a.x += q.x; a.y += q.y; a.z += q.z; a.w += q.w; }
            *reinterpret_cast<float4*>(c + i) = a;
        } else {
            for (size_t j = i; j < n && j < i + 4; ++j) {
                float a = c[j];
                for (int z = 1; z < parts; ++z) a += c[z * stride + j];
                c[j] = a;
            }
        }
    }
}

// z <- cap tanh(z / cap)
static __global__ __launch_bounds__(256) void hy_softcap_kernel(float* __restrict__ z, size_t n, float cap) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) z[i] = cap * tanhf(z[i] / cap);
}

// Per-head products out[t][h][c] = sum_k in[t][h][k] Wt[h][k][c] (float32), optionally times sigmoid(gate[t][h][c]) (gate_mode 2:
// sigmoid(gate[t][h]), one gate per head), for portions of a
// few tokens (decode).  Two uses: the query carried into the latent's space, qa = Wk^T q (scores are then plain dot products with the
// cached latents: q . (Wk c) = (Wk^T q) . c), and the value expansion applied after the weighted sum of latents.  Workgroup = (TT tokens, head, 64 columns): lane =
// column, the four wavefronts split k and meet in LDS, a weight is read once for TT tokens.
template <typename TO, int TT>
static __global__ __launch_bounds__(256) void hy_headmm_kernel(const float* __restrict__ in, int ld_in, int K, int C, const float* __restrict__ Wt,
                                                               const float* __restrict__ gate, int ldg, TO* __restrict__ out, int ldo, int n, int gate_mode = 1) {
    __shared__ float red[3][TT][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, h = blockIdx.y, c = blockIdx.z * 64 + lane, t0 = blockIdx.x * TT;
    const bool livec = c < C;
    float acc[TT];
#pragma unroll
    for (int i = 0; i < TT; ++i) acc[i] = 0.f;
    const float* w = Wt + (size_t)h * K * C + (livec ? c : 0);
    const float* x = in + (size_t)t0 * ld_in + (size_t)h * K;
    // a wavefront takes k in chunks of 8: the chunk's weights and inputs are loaded first, then multiplied (rows past n repeat row 0 and are dropped)
    const float* xr[TT];
#pragma unroll
    for (int i = 0; i < TT; ++i) xr[i] = x + (size_t)(t0 + i < n ? i : 0) * ld_in;
    for (int k0 = wave * 8; k0 < K; k0 += 32) {
        float wv[8], xv[TT][8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int k = min(k0 + u, K - 1);
            wv[u] = k0 + u < K ? w[(size_t)k * C] : 0.f;
#pragma unroll
            for (int i = 0; i < TT; ++i) xv[i][u] = xr[i][k];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int i = 0; i < TT; ++i) acc[i] = fmaf(xv[i][u], wv[u], acc[i]);
    }
    if (wave > 0) {
#pragma unroll
        for (int i = 0; i < TT; ++i) red[wave - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave > 0 || !livec) return;
#pragma unroll
    for (int i = 0; i < TT; ++i) {
        if (t0 + i >= n) break;
        float v = (acc[i] + red[0][i][lane]) + (red[1][i][lane] + red[2][i][lane]);
        if (gate) v *= hy_sigmoid(gate[(size_t)(t0 + i) * ldg + (gate_mode == 2 ? h : h * C + c)]);
        hy_st(out + (size_t)(t0 + i) * ldo + h * C + c, v);
    }
}

// ---- attention core -----------------------------------------------------------------------------------------------------------
// Workgroup = (4 wavefronts, key / value head g, key split).  The rows that share g — (token, head of the group), token-major — are dealt
// out RW at a time; a wavefront owns its RW rows for the whole key loop: running maximum, denominator and DVL x 64 value columns per row in
// registers (rows of different tokens differ only in the position up to which they see keys).  Key tiles of 64 rows are
// staged in LDS (keys padded to an odd stride: a lane reads one key row element by element); lane = key for the scores, lane = value
// column for the weighted sum.  Splits write (max, denominator, unnormalised sum) per (token, head, split); hy_attn_merge_kernel
// joins them, adds the optional extra unit of the denominator and the output gate.
struct HyAttnArgs {
    const float* q; int ldq;            // q of (t, h): q + t ldq + h dk
    const float* kc; const float* vc;   // slot-relative cache bases; row j of head g: kc + j G dk + g dk, vc + j G dv + g dv
    size_t slot_stride;
    int H, G, dk, dv;
    float scale, slope_log2;            // slope_log2 = 0: no distance term
    const int* dyn; int n, nsplit;
    float* part_acc; float* part_ml;    // [n][H][nsplit][dv], [n][H][nsplit][2]
    int kt;                             // keys per tile: 64, or 32 / 16 / 8 where 64 rows do not fit LDS (lanes >= kt idle in the score phase)
    int shared_kv;                      // keys and values are the same rows (latent attention): staged once
    int window, keep;                   // query at position i sees key j <= i if i - j < window or j < keep; window <= 0: every earlier key
    // pool > 0 (with a window): pooled rows pk / pv (laid out like kc / vc, one row per block of `pool` positions); query i also sees
    // the pooled rows of blocks b with b pool + pool - 1 <= i - window
    const float* pk; const float* pv; int pool;
};
constexpr int HY_KT = 64;

// rows j0 .. j0 + KT - 1 of a cache (width floats each, row stride ld) -> LDS rows of stride ls; rows past `last` are zero.  Four
// 16-byte loads are in flight per thread before their LDS stores (width, ld and the base must allow 16-byte loads, else element-wise).
__device__ __forceinline__ void hy_stage_rows(float* __restrict__ dst, int ls, const float* __restrict__ src, int ld, int width, int j0, int KT, int last, bool vec) {
    const int tid = threadIdx.x;
    if (vec) {
        const int cpr = width >> 2, total = KT * cpr;
        for (int i0 = tid; i0 < total; i0 += 4 * 256) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = i0 + u * 256, j = i / cpr, c = i - j * cpr;
                v[u] = (i < total && j0 + j <= last) ? *reinterpret_cast<const float4*>(src + (size_t)(j0 + j) * ld + 4 * c) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int i = i0 + u * 256, j = i / cpr, c = i - j * cpr;
                if (i < total) { float* d = dst + j * ls + 4 * c; d[0] = v[u].x; d[1] = v[u].y; d[2] = v[u].z; d[3] = v[u].w; }
            }
        }
    } else {
        for (int i = tid; i < KT * width; i += 256) {
            const int j = i / width, d = i - j * width;
            dst[j * ls + d] = (j0 + j <= last) ? src[(size_t)(j0 + j) * ld + d] : 0.f;
        }
    }
}

template <int RW, int DVL>
static __global__ __launch_bounds__(256) void hy_attn_kernel(HyAttnArgs a) {
    extern __shared__ float smem[];
    const int dk = a.dk, dv = a.dv, ks = dk | 1;           // odd key stride
    const int KT = a.kt, vs = a.shared_kv ? ks : dv;        // value row stride in LDS
    float* sK = smem;                                       // [KT][ks]
    float* sV = a.shared_kv ? sK : sK + KT * ks;            // [KT][dv]
    float* sQ = sK + KT * ks + (a.shared_kv ? 0 : KT * dv); // [4][dk][RW]
    float* sP = sQ + 4 * dk * RW;                           // [4][KT][RW]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // blockIdx.x = (row block, key / value head) with the LAST row block first: late tokens see the most keys, and workgroups are
    // handed out in index order, so the long ones start first and the short ones fill the gaps they leave
    const int g = blockIdx.x % a.G, rb = (int)(gridDim.x / a.G) - 1 - (int)(blockIdx.x / a.G), split = blockIdx.z, hpg = a.H / a.G;
    // rows of this key / value head: (token, head of the group), token-major; a wavefront owns RW consecutive rows
    const int rows = a.n * hpg, row0 = (rb * 4 + wave) * RW;
    const int pos0 = a.dyn[0];
    const int maxpos = pos0 + min(rows - 1, rb * 4 * RW + 4 * RW - 1) / hpg;      // last key any row of the workgroup sees
    int tr[RW], hr[RW], pr[RW];                            // token, head, position (-1: no such row)
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        const int rho = row0 + r;
        tr[r] = rho < rows ? rho / hpg : 0;
        hr[r] = g * hpg + (rho < rows ? rho % hpg : 0);
        pr[r] = rho < rows ? pos0 + tr[r] : -1;
    }
    const int pos_hi = row0 < rows ? pos0 + min(rows - 1, row0 + RW - 1) / hpg : -1;     // rows ascend: the wavefront's last live row sees the most
    const size_t slot = (size_t)a.dyn[1] * a.slot_stride;
    const float* kc = a.kc + slot + (size_t)g * dk;
    const float* vc = a.vc + slot + (size_t)g * dv;
    const int ldk = a.G * dk, ldv = a.G * dv;
    const bool veck = (dk & 3) == 0 && ((uintptr_t)kc & 15) == 0, vecv = (dv & 3) == 0 && ((uintptr_t)vc & 15) == 0;
    float* myQ = sQ + wave * dk * RW;
    float* myP = sP + wave * KT * RW;
    for (int i = lane; i < dk * RW; i += 64) {
        const int d = i / RW, r = i % RW, rho = row0 + r;
        myQ[i] = rho < rows ? a.q[(size_t)(rho / hpg) * a.ldq + (size_t)(g * hpg + rho % hpg) * dk + d] * a.scale : 0.f;
    }
    float slope[RW], m[RW], l[RW], acc[RW][DVL];
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        slope[r] = a.slope_log2 != 0.f ? exp2f(-a.slope_log2 * (float)(hr[r] + 1) / (float)a.H) : 0.f;
        m[r] = -INFINITY; l[r] = 0.f;
#pragma unroll
        for (int c = 0; c < DVL; ++c) acc[r][c] = 0.f;
    }
    // Key tiles the workgroup visits: the tiles that hold the kept first keys, then the tiles from the window of its earliest row to
    // the position of its latest row; the splits deal this list out in turn.
    const int win = a.window > 0 ? a.window : 0x3fffffff;
    const int minpos = pos0 + (rb * 4 * RW) / hpg;
    const int lo_t = max(0, minpos - win + 1) / KT, hi_t = maxpos / KT;
    const int nk = min((a.keep + KT - 1) / KT, lo_t);
    const int pos_lo = pos0 + min(rows - 1, row0) / hpg;   // the wavefront's earliest row
    // pooled blocks a position sees: those that end at or before pos - window; the tiles of pooled rows come first in the list
    const int P = a.pool;
    int nbr[RW];
#pragma unroll
    for (int r = 0; r < RW; ++r) nbr[r] = P > 0 ? max(0, pr[r] - win + 1) / P : 0;
    const int nb_wg = P > 0 ? max(0, maxpos - win + 1) / P : 0, nb_hi = P > 0 ? max(0, pos_hi - win + 1) / P : 0;
    const int np_t = (nb_wg + KT - 1) / KT, nv = np_t + nk + hi_t - lo_t + 1;
    const float* pkc = P > 0 ? a.pk + slot + (size_t)g * dk : kc;
    const float* pvc = P > 0 ? a.pv + slot + (size_t)g * dv : vc;
    for (int vt = split; vt < nv; vt += a.nsplit) {
        const bool pooled = vt < np_t;
        const int wt = vt - np_t;
        const int j0 = (pooled ? vt : wt < nk ? wt : lo_t + wt - nk) * KT;
        __syncthreads();                                   // previous tile fully consumed (and sQ written, first time)
        hy_stage_rows(sK, ks, pooled ? pkc : kc, ldk, dk, j0, KT, pooled ? nb_wg - 1 : maxpos, veck);
        if (!a.shared_kv) hy_stage_rows(sV, dv, pooled ? pvc : vc, ldv, dv, j0, KT, pooled ? nb_wg - 1 : maxpos, vecv);
        __syncthreads();
        // uniform per wavefront: no row of it sees a key of this tile
        if (pooled ? j0 >= nb_hi : (j0 > pos_hi || (j0 >= a.keep && j0 + KT <= pos_lo - win + 1))) continue;
        float s[RW];
#pragma unroll
        for (int r = 0; r < RW; ++r) s[r] = 0.f;
        const float* kr = sK + (lane < KT ? lane : 0) * ks;
        // eight key elements at a time: their LDS reads are issued together, then multiplied (an element-by-element loop waits for
        // one LDS round trip per element)
        int d = 0;
        for (; d + 8 <= dk; d += 8) {
            float kv[8], qv[8][RW];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                kv[u] = kr[d + u];
#pragma unroll
                for (int r = 0; r < RW; ++r) qv[u][r] = myQ[(d + u) * RW + r];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u)
#pragma unroll
                for (int r = 0; r < RW; ++r) s[r] = fmaf(kv[u], qv[u][r], s[r]);
        }
        for (; d < dk; ++d) {
            const float kv = kr[d];
#pragma unroll
            for (int r = 0; r < RW; ++r) s[r] = fmaf(kv, myQ[d * RW + r], s[r]);
        }
        const int j = j0 + lane;
#pragma unroll
        for (int r = 0; r < RW; ++r) {
            if (pooled) s[r] = (j < nbr[r] && lane < KT) ? s[r] : -INFINITY;
            else s[r] = (j <= pr[r] && lane < KT && (pr[r] - j < win || j < a.keep)) ? s[r] - slope[r] * (float)(pr[r] - j) : -INFINITY;
            const float mn = fmaxf(m[r], hy_wave_max(s[r]));
            const bool any = mn > -INFINITY;                         // false: this row has seen no key yet (its keys start in a later tile of the split)
            const float corr = any ? expf(m[r] - mn) : 1.f;          // exp(-inf) = 0 the first time
            const float p = any ? expf(s[r] - mn) : 0.f;
            l[r] = l[r] * corr + hy_wave_sum(p);
            m[r] = mn;
#pragma unroll
            for (int c = 0; c < DVL; ++c) acc[r][c] *= corr;
            if (lane < KT) myP[lane * RW + r] = p;
        }
        __builtin_amdgcn_wave_barrier();
        const int jn = min(KT, (pooled ? nb_hi : pos_hi + 1) - j0);
        int jj = 0;
        for (; jj + 4 <= jn; jj += 4) {                     // four keys at a time, reads first
            float pj[4][RW], vv[4][DVL];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
#pragma unroll
                for (int r = 0; r < RW; ++r) pj[u][r] = myP[(jj + u) * RW + r];
#pragma unroll
                for (int c = 0; c < DVL; ++c) { const int col = c * 64 + lane; vv[u][c] = col < dv ? sV[(jj + u) * vs + col] : 0.f; }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int c = 0; c < DVL; ++c)
#pragma unroll
                    for (int r = 0; r < RW; ++r) acc[r][c] = fmaf(pj[u][r], vv[u][c], acc[r][c]);
        }
        for (; jj < jn; ++jj) {
            float pj[RW];
#pragma unroll
            for (int r = 0; r < RW; ++r) pj[r] = myP[jj * RW + r];
#pragma unroll
            for (int c = 0; c < DVL; ++c) {
                const int col = c * 64 + lane;
                const float v = col < dv ? sV[jj * vs + col] : 0.f;
#pragma unroll
                for (int r = 0; r < RW; ++r) acc[r][c] = fmaf(pj[r], v, acc[r][c]);
            }
        }
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int r = 0; r < RW; ++r) {
        if (pr[r] < 0) continue;
        const size_t o = ((size_t)tr[r] * a.H + hr[r]) * a.nsplit + split;
        if (lane == 0) { a.part_ml[2 * o] = m[r]; a.part_ml[2 * o + 1] = l[r]; }
#pragma unroll
        for (int c = 0; c < DVL; ++c) {
            const int col = c * 64 + lane;
            if (col < dv) a.part_acc[o * dv + col] = acc[r][c];
        }
    }
}

// out[t][h dv + c] = out_mul * gate * sum_s e^(m_s - M) acc_s[c] / (sum_s e^(m_s - M) l_s + sink e^(z - M)),  M = max(m_s, sink ? z : -inf),
// z = sink_w ? sink_w[h] : 0 (a learned logit per head, or one plain unit).
// gate_mode 1: gate[t][h dv + c], 2: gate[t][h] (one per head).  v_freq != null: the head's output is turned back by the token's
// position over all dv entries (pairs c, c + dv / 2, angle -pos v_freq[c]) before the gate.
template <typename TO>
static __global__ __launch_bounds__(64) void hy_attn_merge_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, int H, int dv, int nsplit,
                                                                  int sink, const float* __restrict__ gate, int ldg, int gate_mode, TO* __restrict__ out, int ldo,
                                                                  const float* __restrict__ v_freq, const int* __restrict__ dyn,
                                                                  const float* __restrict__ sink_w = nullptr, float out_mul = 1.f) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const size_t o = ((size_t)t * H + h) * nsplit;
    const float z = sink_w ? sink_w[h] : 0.f;
    float M = sink ? z : -INFINITY;
    for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[2 * (o + s)]);
    float den = sink ? expf(z - M) : 0.f;
    for (int s = 0; s < nsplit; ++s) {
        const float ms = part_ml[2 * (o + s)];
        if (ms > -INFINITY) den += expf(ms - M) * part_ml[2 * (o + s) + 1];
    }
    auto column = [&](int c) {
        float v = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float ms = part_ml[2 * (o + s)];
            if (ms > -INFINITY) v = fmaf(expf(ms - M), part_acc[(o + s) * dv + c], v);
        }
        return v / den;
    };
    const float ghead = (gate && gate_mode == 2) ? hy_sigmoid(gate[(size_t)t * ldg + h]) : 1.f;
    auto put = [&](int c, float v) {
        if (gate && gate_mode != 2) v *= hy_sigmoid(gate[(size_t)t * ldg + h * dv + c]);
        hy_st(out + (size_t)t * ldo + h * dv + c, v * ghead * out_mul);
    };
    if (v_freq) {
        const int half = dv >> 1;
        const float pos = (float)(dyn[0] + t);
        for (int c = lane; c < half; c += 64) {
            float sn, cs;
            sincosf(pos * v_freq[c], &sn, &cs);
            const float u = column(c), v = column(c + half);
            put(c, u * cs + v * sn);
            put(c + half, v * cs - u * sn);
        }
    } else {
        for (int c = lane; c < dv; c += 64) put(c, column(c));
    }
}

// ---- state-space mixer ------------------------------------------------------------------------------------------------------------
// Causal depthwise convolution over the step's tokens; inputs before the step come from the slot's tail (the last taps - 1 inputs of
// the sequence), zeros before position 0.  out = silu(bias + sum_k w[c][k] in(t - (taps - 1 - k))).
static __global__ __launch_bounds__(256) void hy_conv_kernel(const float* __restrict__ proj, int ld, int x_off, int ch, int taps, const float* __restrict__ w,
                                                             const float* __restrict__ bias, const float* __restrict__ tail, size_t slot_stride,
                                                             const int* __restrict__ dyn, int n, float* __restrict__ out) {
    const int c = blockIdx.x * 256 + threadIdx.x, t = blockIdx.y;
    if (c >= ch) return;
    const bool fresh = dyn[0] == 0;
    const float* tl = tail + (size_t)dyn[1] * slot_stride;
    float a = bias[c];
    for (int k = 0; k < taps; ++k) {
        const int tau = t - (taps - 1 - k);
        const float v = tau >= 0 ? proj[(size_t)tau * ld + x_off + c] : (fresh ? 0.f : tl[(size_t)(taps - 1 + tau) * ch + c]);
        a = fmaf(w[(size_t)c * taps + k], v, a);
    }
    out[(size_t)t * ch + c] = hy_silu(a);
}
// new tail[i] = input at step-relative time n + i - (taps - 1); one thread per channel, ascending i (reads only rows not yet rewritten)
static __global__ __launch_bounds__(256) void hy_conv_tail_kernel(const float* __restrict__ proj, int ld, int x_off, int ch, int taps, float* __restrict__ tail,
                                                                  size_t slot_stride, const int* __restrict__ dyn, int n) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= ch) return;
    const bool fresh = dyn[0] == 0;
    float* tl = tail + (size_t)dyn[1] * slot_stride;
    for (int i = 0; i < taps - 1; ++i) {
        const int tau = n + i - (taps - 1);
        tl[(size_t)i * ch + c] = tau >= 0 ? proj[(size_t)tau * ld + x_off + c] : (fresh ? 0.f : tl[(size_t)(taps - 1 + tau) * ch + c]);
    }
}

// Recurrence S_t = a_t S_(t-1) + b_t k_t x_t^T,  y_t = S_t^T q_t + D x_t  per head, S = N x P (keys / queries of N entries, values of P).
// Three sources of a_t, b_t (HyScanArgs.mode): 0, a state-space layer: dt = softplus(raw + bias), a = e^(-e^(A_log) dt), b = dt, keys
// and queries shared by the heads of a group; 1, gates that a kernel before this one left per (token, head) (hy_mem_gates_kernel);
// 2, a fixed decay per head, b = 1.  Keys, queries and x may pass through silu on the way into LDS (act); keys and queries are
// multiplied by k_mul / q_mul there and may turn by their
// position (rot: first `dims` entries, pairs (i, i + dims / 2) or (2 i, 2 i + 1), angle = position * freq[i]).  ones_col: the last of
// the P columns has x = 1 whatever the token (it then carries n_t = a n + b k, the normaliser of a matrix memory, and y's last column
// is n_t . q_t).
// Workgroup = one head x 4 wavefronts; a wavefront = 64 / NG value columns, a column's N states spread over NG lanes (lane i holds the NL
// states n = i NL .. i NL + NL - 1, in registers for the whole portion; NG NL >= N).  Tokens run in order, TB at a time: the block's key and
// query rows (padded to NG NL), its x columns, a and b are staged in LDS by all four wavefronts (coalesced); every wavefront then
// walks the TB tokens reading its key / query slice with 16-byte LDS reads and leaves its lanes' partial sums of y in LDS; the sums over a
// column's NG lanes, the skip term and the (coalesced) store of y follow once per block, off the recurrence's critical path.  The slot's
// state is read at the start (zero at position 0) and written at the end.
struct HyScanRot { int dims; const float* freq; int interleaved; };
struct HyScanArgs {
    const float* ksrc; int ldk, k_off, k_hstride;      // key of (t, head): ksrc + t ldk + k_off + (head / heads-per-group) k_hstride
    const float* qsrc; int ldq, q_off, q_hstride;
    const float* xsrc; int ldx, x_off;                 // x of (t, head, column): xsrc + t ldx + x_off + head Px + column, Px = P - ones_col
    float k_mul, q_mul;
    int act;                                           // 1: keys, queries and x are silu(source) (before the multipliers)
    HyScanRot rot;
    int mode;
    const float* dtsrc; int ld_dt, dt_off; const float* dt_bias; const float* A_log; const float* Dp;      // mode 0 (Dp: null = no skip term)
    const float* ga; const float* gb;                  // mode 1: [n][heads]
    const float* decay;                                // mode 2: [heads]
    int ones_col;
    int heads, P, N, G, NG, TB;
    float* state; size_t slot_stride; const int* dyn; int n;
    float* y; int ldy;                                 // y of (t, head, column): y + t ldy + head P + column
};
// rows t0 .. t0 + tb - 1 (N floats each, row stride ld) times mul -> dst[t Ns + n], zero behind N; eight loads in flight per thread
__device__ __forceinline__ void hy_scan_stage(float* __restrict__ dst, const float* __restrict__ base, int ld, int t0, int tb, int N, int Ns, float mul, int act) {
    const int total = tb * Ns;
    for (int i0 = threadIdx.x; i0 < total; i0 += 8 * 256) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * 256, t = i / Ns, nn = i - t * Ns;
            v[u] = (i < total && nn < N) ? base[(size_t)(t0 + t) * ld + nn] : 0.f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * 256;
            if (i < total) dst[i] = (act ? hy_silu(v[u]) : v[u]) * mul;
        }
    }
}
// the staged rows turn in place by their position: one thread per pair
__device__ __forceinline__ void hy_scan_turn(float* __restrict__ rows, int tb, int Ns, const HyScanRot& rot, int pos) {
    const int half = rot.dims >> 1;
    for (int i = threadIdx.x; i < tb * half; i += 256) {
        const int t = i / half, j = i - t * half;
        const int i0 = rot.interleaved ? 2 * j : j, i1 = rot.interleaved ? 2 * j + 1 : j + half;
        float sn, cs;
        sincosf((float)(pos + t) * rot.freq[j], &sn, &cs);
        float* r = rows + t * Ns;
        const float u = r[i0], v = r[i1];
        r[i0] = u * cs - v * sn;
        r[i1] = v * cs + u * sn;
    }
}
template <int NL>
static __global__ __launch_bounds__(256) void hy_ssm_scan_kernel(HyScanArgs a) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    const int P = a.P, N = a.N, NG = a.NG, TB = a.TB, n = a.n, Px = P - (a.ones_col ? 1 : 0);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, head = blockIdx.y, ng = lane % NG;
    const int cpw = 64 / NG, cols = 4 * cpw, col0 = blockIdx.x * cols, myc = wave * cpw + lane / NG, p = col0 + myc, Ns = NG * NL;
    const bool livep = p < P;
    const int g = head / (a.heads / a.G);
    const float* kbase = a.ksrc + a.k_off + (size_t)g * a.k_hstride;
    const float* qbase = a.qsrc + a.q_off + (size_t)g * a.q_hstride;
    const float* xbase = a.xsrc + a.x_off + (size_t)head * Px;
    float* sB = smem;                    // [TB][Ns]
    float* sC = sB + TB * Ns;            // [TB][Ns]
    float* sY = sC + TB * Ns;            // [TB][256] partial sums of y per lane
    float* sX = sY + TB * 256;           // [TB][cols]
    float* sDt = sX + TB * cols;         // [TB] b_t, [TB] a_t
    float* S = a.state + (size_t)a.dyn[1] * a.slot_stride + (size_t)head * N * P;
    const int pos0 = a.dyn[0];
    const bool fresh = pos0 == 0;
    float s[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int nn = ng * NL + i;
        s[i] = (!fresh && livep && nn < N) ? S[(size_t)nn * P + p] : 0.f;
    }
    const float na = a.mode == 0 ? -expf(a.A_log[head]) : 0.f, dtb = a.mode == 0 ? a.dt_bias[head] : 0.f, dd = (a.mode == 0 && a.Dp) ? a.Dp[head] : 0.f;
    const float fixed = a.mode == 2 ? a.decay[head] : 0.f;
    for (int t0 = 0; t0 < n; t0 += TB) {
        const int tb = min(TB, n - t0);
        __syncthreads();
        hy_scan_stage(sB, kbase, a.ldk, t0, tb, N, Ns, a.k_mul, a.act);
        hy_scan_stage(sC, qbase, a.ldq, t0, tb, N, Ns, a.q_mul, a.act);
        for (int i = tid; i < tb * cols; i += 256) {
            const int t = i / cols, c = i - t * cols;
            if (col0 + c < Px) { const float xv = xbase[(size_t)(t0 + t) * a.ldx + col0 + c]; sX[i] = a.act ? hy_silu(xv) : xv; }
            else sX[i] = col0 + c < P ? 1.f : 0.f;
        }
        if (tid < tb) {
            if (a.mode == 0) {
                const float dt = hy_softplus(a.dtsrc[(size_t)(t0 + tid) * a.ld_dt + a.dt_off + head] + dtb);
                sDt[tid] = dt;
                sDt[TB + tid] = expf(na * dt);
            } else if (a.mode == 1) {
                sDt[tid] = a.gb[(size_t)(t0 + tid) * a.heads + head];
                sDt[TB + tid] = a.ga[(size_t)(t0 + tid) * a.heads + head];
            } else {
                sDt[tid] = 1.f;
                sDt[TB + tid] = fixed;
            }
        }
        if (a.rot.dims > 0) {          // a turn is linear: the multiplier went in with the staging
            __syncthreads();
            hy_scan_turn(sB, tb, Ns, a.rot, pos0 + t0);
            hy_scan_turn(sC, tb, Ns, a.rot, pos0 + t0);
        }
        __syncthreads();
        for (int t = 0; t < tb; ++t) {
            const float dx = sDt[t] * sX[t * cols + myc], decay = sDt[TB + t];
            const float4* b4 = reinterpret_cast<const float4*>(sB + t * Ns + ng * NL);
            const float4* c4 = reinterpret_cast<const float4*>(sC + t * Ns + ng * NL);
            float a0 = 0.f, a1 = 0.f;
#pragma unroll
            for (int q = 0; q < NL / 4; ++q) {
                const float4 bv = b4[q], cv = c4[q];
                s[4 * q] = fmaf(decay, s[4 * q], bv.x * dx);         a0 = fmaf(s[4 * q], cv.x, a0);
                s[4 * q + 1] = fmaf(decay, s[4 * q + 1], bv.y * dx); a1 = fmaf(s[4 * q + 1], cv.y, a1);
                s[4 * q + 2] = fmaf(decay, s[4 * q + 2], bv.z * dx); a0 = fmaf(s[4 * q + 2], cv.z, a0);
                s[4 * q + 3] = fmaf(decay, s[4 * q + 3], bv.w * dx); a1 = fmaf(s[4 * q + 3], cv.w, a1);
            }
            sY[t * 256 + tid] = a0 + a1;
        }
        __syncthreads();
        for (int i = tid; i < tb * cols; i += 256) {
            const int t = i / cols, c = i - t * cols;
            if (col0 + c >= P) continue;
            float v = 0.f;
            for (int k = 0; k < NG; ++k) v += sY[t * 256 + c * NG + k];
            a.y[(size_t)(t0 + t) * a.ldy + head * P + col0 + c] = fmaf(dd, sX[i], v);
        }
    }
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        const int nn = ng * NL + i;
        if (livep && nn < N) S[(size_t)nn * P + p] = s[i];
    }
}

// Gates of a matrix memory with exponential gating, per (token, head), from the raw gate projections z_i, z_f (+ biases):
//   i = cap tanh(z_i / cap), f = logsigmoid(cap tanh(z_f / cap)), m_t = max(f + m_(t-1), i) (m before the first token is 0),
//   ga = e^(f + m_(t-1) - m_t), gb = e^(i - m_t), ge = e^(-m_t).
// One workgroup per head: i and f of a block of tokens are made by all threads, one thread walks the chain of maxima (two operations a
// token), all threads finish ga / gb / ge.  The slot keeps m.
constexpr int HY_GATE_TB = 1024;
static __global__ __launch_bounds__(256) void hy_mem_gates_kernel(const float* __restrict__ proj, int ld, int i_off, int f_off, const float* __restrict__ bias, float cap,
                                                                  int heads, float* __restrict__ mstate, size_t slot_stride, const int* __restrict__ dyn, int n,
                                                                  float* __restrict__ ga, float* __restrict__ gb, float* __restrict__ ge) {
    __shared__ float si[HY_GATE_TB], sf[HY_GATE_TB], sm[HY_GATE_TB + 1];
    const int head = blockIdx.x, tid = threadIdx.x;
    float* mp = mstate + (size_t)dyn[1] * slot_stride + head;
    float mprev = dyn[0] == 0 ? 0.f : *mp;
    for (int t0 = 0; t0 < n; t0 += HY_GATE_TB) {
        const int tb = min(HY_GATE_TB, n - t0);
        __syncthreads();
        for (int t = tid; t < tb; t += 256) {
            const float* row = proj + (size_t)(t0 + t) * ld;
            const float zi = row[i_off + head] + (bias ? bias[i_off + head] : 0.f), zf = row[f_off + head] + (bias ? bias[f_off + head] : 0.f);
            si[t] = cap * tanhf(zi / cap);
            const float fr = cap * tanhf(zf / cap);
            sf[t] = fminf(fr, 0.f) - log1pf(expf(-fabsf(fr)));          // log sigmoid
        }
        __syncthreads();
        if (tid == 0) {
            float m = mprev;
            sm[0] = m;
            for (int t = 0; t < tb; ++t) { m = fmaxf(sf[t] + m, si[t]); sm[t + 1] = m; }
        }
        __syncthreads();
        for (int t = tid; t < tb; t += 256) {
            const size_t o = (size_t)(t0 + t) * heads + head;
            ga[o] = expf(sf[t] + sm[t] - sm[t + 1]);
            gb[o] = expf(si[t] - sm[t + 1]);
            ge[o] = expf(-sm[t + 1]);
        }
        mprev = sm[tb];          // every thread reads the same value before the next block's barrier
    }
    if (tid == 0) *mp = mprev;
}

// What leaves a matrix memory: one wavefront per (token, head).  o = y[0 .. V) of the head (row stride ldy, P = V or V + 1 columns per
// head), divided by max(|y[V]|, ge[t][head]) + 1e-6 where the memory has a normaliser (ge != null); then o / sqrt(mean(o^2) + eps), times
// w[head V + c] (null = none), times act(gate[t][g_off + head V + c]) (act = silu, or sigmoid for gate_act 1), times out_mul, stored in the
// matrix type at out[t ldo + head V + c].
// NT threads per (token, head): 64 for portions of many tokens, 256 for a few (a thread's column loop is a chain of load round trips).
template <typename TO, int NT>
static __global__ __launch_bounds__(NT) void hy_mem_out_kernel(const float* __restrict__ y, int ldy, int P, int V, const float* __restrict__ ge, int heads,
                                                               const float* __restrict__ w, const float* __restrict__ gate, int ldg, int g_off, int gate_act,
                                                               float eps, float out_mul, TO* __restrict__ out, int ldo) {
    __shared__ float red[NT / 64];
    const int t = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const float* row = y + (size_t)t * ldy + (size_t)head * P;
    float inv = 1.f;
    if (ge) inv = 1.f / (fmaxf(fabsf(row[V]), ge[(size_t)t * heads + head]) + 1e-6f);
    // the first two columns of a thread stay in registers with their gate and weight (loaded before the sum's barrier)
    float keep[2], kz[2], kw[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int c = tid + u * NT;
        keep[u] = c < V ? row[c] * inv : 0.f;
        kz[u] = c < V ? gate[(size_t)t * ldg + g_off + head * V + c] : 0.f;
        kw[u] = (c < V && w) ? w[head * V + c] : 1.f;
    }
    float ss = keep[0] * keep[0] + keep[1] * keep[1];
    for (int c = tid + 2 * NT; c < V; c += NT) { const float v = row[c] * inv; ss += v * v; }
    if constexpr (NT == 64) ss = hy_wave_sum(ss);
    else ss = hy_block_sum<NT>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)V + eps);
#pragma unroll
    for (int u = 0; u < 2; ++u) {
        const int c = tid + u * NT;
        if (c < V) hy_st(out + (size_t)t * ldo + head * V + c, keep[u] * r * kw[u] * (gate_act == 1 ? hy_sigmoid(kz[u]) : hy_silu(kz[u])) * out_mul);
    }
    for (int c = tid + 2 * NT; c < V; c += NT) {
        const float z = gate[(size_t)t * ldg + g_off + head * V + c];
        const float gv = gate_act == 1 ? hy_sigmoid(z) : hy_silu(z);
        hy_st(out + (size_t)t * ldo + head * V + c, row[c] * inv * r * (w ? w[head * V + c] : 1.f) * gv * out_mul);
    }
}

// y * silu(z), unit root mean square per part (ngroups equal parts of inner), times the weight
template <typename TO>
static __global__ __launch_bounds__(256) void hy_gated_norm_kernel(const float* __restrict__ y, const float* __restrict__ proj, int ld, int z_off, int inner,
                                                                   int ngroups, const float* __restrict__ w, float eps, TO* __restrict__ out, int ldo) {
    __shared__ float red[4];
    const int t = blockIdx.x, grp = blockIdx.y, len = inner / ngroups, c0 = grp * len;
    float ss = 0.f;
    for (int i = threadIdx.x; i < len; i += 256) {
        const float v = y[(size_t)t * inner + c0 + i] * hy_silu(proj[(size_t)t * ld + z_off + c0 + i]);
        ss += v * v;
    }
    ss = hy_block_sum<256>(ss, red);
    const float r = 1.f / sqrtf(ss / (float)len + eps);
    for (int i = threadIdx.x; i < len; i += 256) {
        const float v = y[(size_t)t * inner + c0 + i] * hy_silu(proj[(size_t)t * ld + z_off + c0 + i]);
        hy_st(out + (size_t)t * ldo + c0 + i, v * r * w[c0 + i]);
    }
}
