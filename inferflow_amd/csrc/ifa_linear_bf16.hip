// ifa_linear_bf16.hip -- linear layers with bfloat16 weights [N][K] and 32-bit activations [T][K]:
//   C[t][n] (+)= alpha * mul[n] * act(sum_k A[t][k] W[n][k] + bias[n])     (mul, bias optional; act = SiLU on a column range, else identity;
//                                                                          C in 32-bit floats)
// The epilogue covers a plain projection (store), a projection with bias, and the residual update of a layer
// (accumulate into the 32-bit residual stream with a per-channel layer scale and a branch scale).
//
//   T <= 8    k_lin_rows: one wave per output row, the weight row streamed once in 16-byte pieces, all T activation rows
//             multiplied against it in fp32 (decode steps: bound by the weight stream)
//   T  > 8    k_lin_mfma: 64 x 64 output tiles, K in steps of 32 through LDS, four waves of 32 x 32 sub-tiles;
//             OPS32 = false: operands rounded to bfloat16, v_mfma_f32_32x32x16_bf16;
//             OPS32 = true : operands stay 32-bit, v_mfma_f32_32x32x2_f32 (the exact mode of the worker)
// Accumulation is fp32 in every path.  No atomics, no split K: a result does not depend on what else runs.
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"

using namespace ifa32;

namespace {

typedef float f32x16v __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

struct LinArgs {
    const bf16_t *W; const float *A; float *C;
    const bf16_t *bias, *mul;
    int T, N, K, lda, ldc;
    float alpha; int accumulate, vec;
    int act_c0, act_c1;          // output columns [act_c0, act_c1) pass SiLU after the bias (projections whose consumer wants them activated)
    const bf16_t *norm_w; float norm_eps;      // row kernel, prologue 1: the activations are layer-normed (no bias) on the fly
    // grouped product (k_lin_mfma only): tile blockIdx.y serves rows [row0, row0 + n) of group g (tile_map {g, row0, n}; *n_tiles valid
    // tiles) with the matrix W + g * N * K; activation row of output row r: A[a_rows[r]] (a_rows null: r); row_scale per output row
    const int *tile_map, *n_tiles, *a_rows; const float *row_scale;
    int act_kind;                              // 1: every output passes the exact (erf) GELU after the bias
};

__device__ __forceinline__ void lin_store(const LinArgs &P, int t, int n, float acc)
{
    if (P.bias) acc += bf2f(P.bias[n]);
    if (n >= P.act_c0 && n < P.act_c1) acc = silu_exact(acc);
    if (P.act_kind == 1) acc = 0.5f * acc * (1.0f + erff(acc * 0.70710678118654752f));
    if (P.row_scale) acc *= P.row_scale[t];
    if (P.mul) acc *= bf2f(P.mul[n]);
    acc *= P.alpha;
    float *c = P.C + (size_t)t * P.ldc + n;
    *c = P.accumulate ? *c + acc : acc;
}

constexpr int LM_T = 64, LM_N = 64, LM_K = 32;

template <bool OPS32>
__global__ void __launch_bounds__(256) k_lin_mfma(LinArgs P)
{
    // bf16 operands: [64][40] halfs per matrix (row stride 80 bytes: 16-byte aligned fragments);
    // 32-bit operands: [64][33] floats per matrix
    __shared__ __attribute__((aligned(16))) char smem[OPS32 ? 2 * LM_T * 33 * 4 : 2 * LM_T * 40 * 2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 31, g = lane >> 5;
    const int wm = wave & 1, wn = wave >> 1;
    int t0 = blockIdx.y * LM_T, t_end = P.T;
    const int n0 = blockIdx.x * LM_N;
    const bf16_t *Wg = P.W;
    if (P.tile_map) {
        if ((int)blockIdx.y >= *P.n_tiles) return;
        const int *tm = P.tile_map + 3 * blockIdx.y;
        Wg += (size_t)tm[0] * P.N * P.K; t0 = tm[1]; t_end = tm[1] + tm[2];
    }
    const int lr = tid >> 2, lc = (tid & 3) * 8;      // this thread stages 8 consecutive k of row lr
    const size_t a_row = (t0 + lr < t_end) ? (size_t)(P.a_rows ? P.a_rows[t0 + lr] : t0 + lr) : 0;
    f32x16v acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.0f;

    for (int k0 = 0; k0 < P.K; k0 += LM_K) {
        float a8[8], w8[8];
        {
            const int t = t0 + lr, n = n0 + lr, k = k0 + lc;
            const bool in_a = t < t_end, in_w = n < P.N;
            if (P.vec && k + 8 <= P.K) {
                if (in_a) {
                    const float4 v0 = *reinterpret_cast<const float4 *>(P.A + a_row * P.lda + k);
                    const float4 v1 = *reinterpret_cast<const float4 *>(P.A + a_row * P.lda + k + 4);
                    a8[0] = v0.x; a8[1] = v0.y; a8[2] = v0.z; a8[3] = v0.w; a8[4] = v1.x; a8[5] = v1.y; a8[6] = v1.z; a8[7] = v1.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) a8[e] = 0.0f;
                }
                if (in_w) {
                    const u32x4v wv = *reinterpret_cast<const u32x4v *>(Wg + (size_t)n * P.K + k);
#pragma unroll
                    for (int e = 0; e < 4; e++) { w8[2 * e] = __uint_as_float(wv[e] << 16); w8[2 * e + 1] = __uint_as_float(wv[e] & 0xFFFF0000u); }
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) w8[e] = 0.0f;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const bool kin = k + e < P.K;
                    a8[e] = in_a && kin ? P.A[a_row * P.lda + k + e] : 0.0f;
                    w8[e] = in_w && kin ? bf2f(Wg[(size_t)n * P.K + k + e]) : 0.0f;
                }
            }
        }
        __syncthreads();      // the previous step's fragments have been read
        if constexpr (OPS32) {
            float *As = reinterpret_cast<float *>(smem), *Ws = As + LM_T * 33;
#pragma unroll
            for (int e = 0; e < 8; e++) { As[lr * 33 + lc + e] = a8[e]; Ws[lr * 33 + lc + e] = w8[e]; }
        } else {
            bf16_t *As = reinterpret_cast<bf16_t *>(smem), *Ws = As + LM_T * 40;
            u32x4v av, wv;
#pragma unroll
            for (int e = 0; e < 4; e++) {
                av[e] = (uint32_t)f2bf(a8[2 * e]) | ((uint32_t)f2bf(a8[2 * e + 1]) << 16);
                wv[e] = (__float_as_uint(w8[2 * e]) >> 16) | (__float_as_uint(w8[2 * e + 1]) & 0xFFFF0000u);
            }
            *reinterpret_cast<u32x4v *>(As + lr * 40 + lc) = av;
            *reinterpret_cast<u32x4v *>(Ws + lr * 40 + lc) = wv;
        }
        __syncthreads();
        if constexpr (OPS32) {
            const float *As = reinterpret_cast<const float *>(smem), *Ws = As + LM_T * 33;
#pragma unroll
            for (int s = 0; s < LM_K / 2; s++)
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(As[(32 * wm + i) * 33 + 2 * s + g], Ws[(32 * wn + i) * 33 + 2 * s + g], acc, 0, 0, 0);
        } else {
            const bf16_t *As = reinterpret_cast<const bf16_t *>(smem), *Ws = As + LM_T * 40;
#pragma unroll
            for (int s = 0; s < LM_K / 16; s++) {
                const bf16x8v af = __builtin_bit_cast(bf16x8v, *reinterpret_cast<const u32x4v *>(As + (32 * wm + i) * 40 + 16 * s + 8 * g));
                const bf16x8v wf = __builtin_bit_cast(bf16x8v, *reinterpret_cast<const u32x4v *>(Ws + (32 * wn + i) * 40 + 16 * s + 8 * g));
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, wf, acc, 0, 0, 0);
            }
        }
    }
    const int n = n0 + 32 * wn + i;
    if (n < P.N) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int t = t0 + 32 * wm + (r & 3) + 8 * (r >> 2) + 4 * g;
            if (t < t_end) lin_store(P, t, n, acc[r]);
        }
    }
}

// T <= TT rows; one wave per output row at a time.  PRO: what the activations pass as they are read (steps of a few rows are bound
// by launches and dependent loads, not arithmetic, so the neighbouring element-wise launch is folded in here):
//   1  layer norm without bias: a = (x - mean) / sqrt(var + eps) * w[k]   (every wave forms mean and variance of the T rows itself)
//   2  gated GELU: the row holds gate | up (2 K values), a = gelu_tanh(gate[k]) * up[k]
template <int TT, int PRO>
__global__ void __launch_bounds__(256) k_lin_rows(LinArgs P)
{
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), nwaves = gridDim.x * (blockDim.x >> 6);
    float mean[TT], rstd[TT];
    if (PRO == 1) {
#pragma unroll
        for (int t = 0; t < TT; t++) {
            const float *a = P.A + (size_t)min(t, P.T - 1) * P.lda;
            float s = 0.0f;
            for (int k = lane * 4; k < P.K; k += 256) { const float4 v = *reinterpret_cast<const float4 *>(a + k); s += (v.x + v.y) + (v.z + v.w); }
            mean[t] = wave_sum(s) / (float)P.K;
            float q = 0.0f;
            for (int k = lane * 4; k < P.K; k += 256) {
                const float4 v = *reinterpret_cast<const float4 *>(a + k);
                const float d0 = v.x - mean[t], d1 = v.y - mean[t], d2 = v.z - mean[t], d3 = v.w - mean[t];
                q += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
            }
            rstd[t] = 1.0f / sqrtf(wave_sum(q) / (float)P.K + P.norm_eps);
        }
    }
    for (int n = wave; n < P.N; n += nwaves) {
        float acc[TT];
#pragma unroll
        for (int t = 0; t < TT; t++) acc[t] = 0.0f;
        const bf16_t *w = P.W + (size_t)n * P.K;
        if (P.vec) {
            for (int k = lane * 8; k < P.K; k += 512) {
                const u32x4v wv = *reinterpret_cast<const u32x4v *>(w + k);
                float w8[8], g8[8];
#pragma unroll
                for (int e = 0; e < 4; e++) { w8[2 * e] = __uint_as_float(wv[e] << 16); w8[2 * e + 1] = __uint_as_float(wv[e] & 0xFFFF0000u); }
                if (PRO == 1) {
                    const u32x4v gv = *reinterpret_cast<const u32x4v *>(P.norm_w + k);
#pragma unroll
                    for (int e = 0; e < 4; e++) { g8[2 * e] = __uint_as_float(gv[e] << 16); g8[2 * e + 1] = __uint_as_float(gv[e] & 0xFFFF0000u); }
                }
#pragma unroll
                for (int t = 0; t < TT; t++) {
                    const float *a = P.A + (size_t)min(t, P.T - 1) * P.lda + k;
                    const float4 v0 = *reinterpret_cast<const float4 *>(a), v1 = *reinterpret_cast<const float4 *>(a + 4);
                    float x8[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                    if (PRO == 1) {
#pragma unroll
                        for (int e = 0; e < 8; e++) x8[e] = (x8[e] - mean[t]) * rstd[t] * g8[e];
                    } else if (PRO == 2) {
                        const float4 u0 = *reinterpret_cast<const float4 *>(a + P.K), u1 = *reinterpret_cast<const float4 *>(a + P.K + 4);
                        const float u8[8] = {u0.x, u0.y, u0.z, u0.w, u1.x, u1.y, u1.z, u1.w};
#pragma unroll
                        for (int e = 0; e < 8; e++) x8[e] = gelu_tanh_f(x8[e]) * u8[e];
                    }
                    float s = acc[t];
#pragma unroll
                    for (int e = 0; e < 8; e++) s = fmaf(x8[e], w8[e], s);
                    acc[t] = s;
                }
            }
        } else {
            for (int k = lane; k < P.K; k += 64) {
                const float wk = bf2f(w[k]);
#pragma unroll
                for (int t = 0; t < TT; t++) acc[t] = fmaf(P.A[(size_t)min(t, P.T - 1) * P.lda + k], wk, acc[t]);
            }
        }
#pragma unroll
        for (int t = 0; t < TT; t++) acc[t] = wave_sum(acc[t]);
#pragma unroll
        for (int t = 0; t < TT; t++)
            if (lane == t && t < P.T) lin_store(P, t, n, acc[t]);
    }
}

} // namespace

static int linear_launch(const void *w_bf16, size_t rows, size_t cols, const void *a_f32, size_t lda, size_t tokens, const void *bias_bf16,
                         const void *mul_bf16, float alpha, int accumulate, int ops32, void *c_f32, size_t ldc, int silu_col0, int silu_col1, int prologue,
                         const void *norm_w_bf16, float norm_eps, ifa_stream stream, const char *who)
{
    IFA_REQUIRE(w_bf16 && a_f32 && c_f32, "%s: null pointer", who);
    IFA_REQUIRE(rows > 0 && cols > 0 && tokens > 0 && lda >= cols * (prologue == 2 ? 2 : 1) && ldc >= rows, "%s: bad shape (%zu x %zu, %zu tokens, lda %zu, ldc %zu)", who, rows, cols, tokens, lda, ldc);
    IFA_REQUIRE(rows < (1u << 30) && cols < (1u << 30) && tokens < (1u << 30), "%s: dimension too large", who);
    LinArgs P;
    P.W = (const bf16_t *)w_bf16; P.A = (const float *)a_f32; P.C = (float *)c_f32;
    P.bias = (const bf16_t *)bias_bf16; P.mul = (const bf16_t *)mul_bf16;
    P.T = (int)tokens; P.N = (int)rows; P.K = (int)cols; P.lda = (int)lda; P.ldc = (int)ldc;
    P.alpha = alpha; P.accumulate = accumulate ? 1 : 0; P.act_c0 = silu_col0; P.act_c1 = silu_col1;
    P.norm_w = (const bf16_t *)norm_w_bf16; P.norm_eps = norm_eps;
    P.tile_map = P.n_tiles = P.a_rows = nullptr; P.row_scale = nullptr; P.act_kind = 0;
    // 16-byte requests need whole 8-element pieces in every row of both operands
    P.vec = (cols % 8 == 0 && lda % 4 == 0 && ((uintptr_t)a_f32 & 15) == 0 && ((uintptr_t)w_bf16 & 15) == 0) ? 1 : 0;
    hipStream_t s = ifa_s(stream);
    if (prologue) {
        IFA_REQUIRE(prologue == 1 || prologue == 2, "%s: prologue %d", who, prologue);
        IFA_REQUIRE(tokens <= 8 && P.vec, "%s: a fused prologue needs at most 8 rows and 16-byte aligned rows of whole 8-element pieces", who);
        IFA_REQUIRE(prologue != 1 || (norm_w_bf16 && ((uintptr_t)norm_w_bf16 & 15) == 0), "%s: the norm's weight is missing or unaligned", who);
    }
    if (tokens <= 8) {
        const unsigned grid = (unsigned)std::min<size_t>((rows + 3) / 4, 8192);
#define IFA_LR(TT) { if (prologue == 1) hipLaunchKernelGGL((k_lin_rows<TT, 1>), dim3(grid), dim3(256), 0, s, P); \
                     else if (prologue == 2) hipLaunchKernelGGL((k_lin_rows<TT, 2>), dim3(grid), dim3(256), 0, s, P); \
                     else hipLaunchKernelGGL((k_lin_rows<TT, 0>), dim3(grid), dim3(256), 0, s, P); }
        if (tokens == 1) IFA_LR(1) else if (tokens == 2) IFA_LR(2) else if (tokens <= 4) IFA_LR(4) else IFA_LR(8)
#undef IFA_LR
    } else {
        const dim3 grid(ifa_cdiv(rows, LM_N), ifa_cdiv(tokens, LM_T));
        if (ops32) hipLaunchKernelGGL(k_lin_mfma<true>, grid, dim3(256), 0, s, P);
        else hipLaunchKernelGGL(k_lin_mfma<false>, grid, dim3(256), 0, s, P);
    }
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

extern "C" int ifa_linear_bf16w(const void *w_bf16, size_t rows, size_t cols, const void *a_f32, size_t lda, size_t tokens,
                                const void *bias_bf16, const void *mul_bf16, float alpha, int accumulate, int ops32,
                                void *c_f32, size_t ldc, int silu_col0, int silu_col1, ifa_stream stream)
{
    return linear_launch(w_bf16, rows, cols, a_f32, lda, tokens, bias_bf16, mul_bf16, alpha, accumulate, ops32, c_f32, ldc, silu_col0, silu_col1, 0, nullptr, 0.0f,
                         stream, "ifa_linear_bf16w");
}

extern "C" int ifa_linear_bf16w_rows(int prologue, const void *norm_w_bf16, float norm_eps, const void *w_bf16, size_t rows, size_t cols, const void *a_f32,
                                     size_t lda, size_t tokens, const void *bias_bf16, const void *mul_bf16, float alpha, int accumulate, void *c_f32,
                                     size_t ldc, int silu_col0, int silu_col1, ifa_stream stream)
{
    IFA_REQUIRE(tokens <= 8, "ifa_linear_bf16w_rows: %zu rows (at most 8)", tokens);
    return linear_launch(w_bf16, rows, cols, a_f32, lda, tokens, bias_bf16, mul_bf16, alpha, accumulate, 1, c_f32, ldc, silu_col0, silu_col1, prologue,
                         norm_w_bf16, norm_eps, stream, "ifa_linear_bf16w_rows");
}

// Grouped product on the matrix cores: `groups` matrices [rows][cols] back to back in w_bf16; the output rows are sorted by group and
// cut into tiles of at most 64 rows of ONE group: tile_map_dev[3 i] = {group, first row, rows}, *n_tiles_dev tiles (max_tiles bounds the
// grid).  C[r][n] = row_scale[r] * act(sum_k A[a_rows[r]][k] W_group[n][k]); a_rows_dev / row_scale_f32 nullable; act 0 none, 1 erf-GELU.
extern "C" int ifa_linear_bf16w_grouped(const void *w_bf16, size_t rows, size_t cols, int groups, const void *a_f32, size_t lda, const int *a_rows_dev,
                                        const int *tile_map_dev, const int *n_tiles_dev, size_t max_tiles, const void *row_scale_f32, int act, int ops32,
                                        void *c_f32, size_t ldc, ifa_stream stream)
{
    IFA_REQUIRE(w_bf16 && a_f32 && c_f32 && tile_map_dev && n_tiles_dev, "ifa_linear_bf16w_grouped: null pointer");
    IFA_REQUIRE(rows > 0 && cols > 0 && groups > 0 && max_tiles > 0 && max_tiles < 65536 && lda >= cols && ldc >= rows && (act == 0 || act == 1), "ifa_linear_bf16w_grouped: bad shape");
    IFA_REQUIRE(rows < (1u << 30) && cols < (1u << 30), "ifa_linear_bf16w_grouped: dimension too large");
    LinArgs P;
    P.W = (const bf16_t *)w_bf16; P.A = (const float *)a_f32; P.C = (float *)c_f32; P.bias = nullptr; P.mul = nullptr;
    P.T = 0; P.N = (int)rows; P.K = (int)cols; P.lda = (int)lda; P.ldc = (int)ldc; P.alpha = 1.0f; P.accumulate = 0; P.act_c0 = P.act_c1 = 0;
    P.norm_w = nullptr; P.norm_eps = 0.0f;
    P.tile_map = tile_map_dev; P.n_tiles = n_tiles_dev; P.a_rows = a_rows_dev; P.row_scale = (const float *)row_scale_f32; P.act_kind = act;
    P.vec = (cols % 8 == 0 && lda % 4 == 0 && ((uintptr_t)a_f32 & 15) == 0 && ((uintptr_t)w_bf16 & 15) == 0 && (rows * cols) % 8 == 0) ? 1 : 0;
    const dim3 grid(ifa_cdiv(rows, LM_N), (unsigned)max_tiles);
    if (ops32) hipLaunchKernelGGL(k_lin_mfma<true>, grid, dim3(256), 0, ifa_s(stream), P);
    else hipLaunchKernelGGL(k_lin_mfma<false>, grid, dim3(256), 0, ifa_s(stream), P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}
