// ifa_attn_latent.hip -- latent attention: every position leaves ONE cache row [kv_rank latent c | rot_dim rotated key part] in
// 32-bit floats that all heads share; a head's unrotated key is W_uk[h] c, its value W_uv[h] c, and
//     score(i, j, h) = (q_u[i][h] . W_uk[h] c_j + q_r[i][h] . k_r[j]) * scale,   causal, ordinary softmax.
// Two forms of the same sums:
//   single tokens   the key map is absorbed into the query, qa[h] = [W_uk[h]^T q_u | q_r], which is then a query of kv_rank + rot_dim
//                   dimensions against the cache rows themselves (one shared "KV head": ifa_attention_window_f32 with the value row =
//                   the key row); the latent result goes through W_uv[h] afterwards.  The cache is read once per head, nothing is expanded.
//   prompts         keys and values of the sequence's positions are expanded by two products over the cached latents
//                   (ifa_linear_bf16w) and k_attn_latent_tile runs 128 queries of one sequence per workgroup on the fp32 matrix
//                   cores, reading the rotated key part straight from the cache rows.
// Rotation: interleaved pairs (2i, 2i + 1) of the first rot_dims dimensions of the rotated part turn by pos * freq[i]; the angle is
// formed in double (at position 1000 one fp32 ulp of an angle is 1e-4).
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"

using namespace ifa32;

namespace {

// one workgroup per row: latent normed into the cache, key part rotated into the cache, the rotated part of every query head in place
__global__ void __launch_bounds__(256) k_latent_prepare(const float *__restrict__ kv, size_t ldkv, int R, int dr, int rdims, const bf16_t *__restrict__ cw, float eps,
                                                        float *__restrict__ q, size_t ldq, int heads, int dim, const double *__restrict__ freq, float mult,
                                                        const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq, float *const *__restrict__ slot_base,
                                                        size_t cache_off)
{
    extern __shared__ float cs[];          // [rdims / 2] cos, [rdims / 2] sin
    __shared__ float red[17];
    const int t = blockIdx.x, tid = threadIdx.x, half = rdims / 2;
    const SeqDesc sd = seqs[row_seq[t]];
    const int pos = sd.pos0 + t - sd.row0;
    for (int i = tid; i < half; i += blockDim.x) {
        const double a = (double)pos * freq[i];
        cs[i] = (float)(cos(a) * (double)mult);
        cs[half + i] = (float)(sin(a) * (double)mult);
    }
    const float *kr = kv + (size_t)t * ldkv;
    float *row = slot_base[sd.slot] + cache_off + (size_t)pos * (R + dr);
    float s = 0.0f;
    for (int c = tid; c < R; c += blockDim.x) s = fmaf(kr[c], kr[c], s);
    const float rinv = 1.0f / sqrtf(block_sum(s, red) / (float)R + eps);          // (the barrier inside also publishes cs)
    for (int c = tid; c < R; c += blockDim.x) row[c] = kr[c] * rinv * bf2f(cw[c]);
    for (int i = tid; i < half; i += blockDim.x) {
        const float u = kr[R + 2 * i], v = kr[R + 2 * i + 1], co = cs[i], si = cs[half + i];
        row[R + 2 * i] = u * co - v * si;
        row[R + 2 * i + 1] = v * co + u * si;
    }
    for (int c = rdims + tid; c < dr; c += blockDim.x) row[R + c] = kr[R + c];
    float *qr = q + (size_t)t * ldq;
    for (int e = tid; e < heads * half; e += blockDim.x) {
        const int h = e / half, i = e % half;
        float *p = qr + (size_t)h * (dim + dr) + dim + 2 * i;
        const float u = p[0], v = p[1], co = cs[i], si = cs[half + i];
        p[0] = u * co - v * si;
        p[1] = v * co + u * si;
    }
}

// grid (rows, heads, chunks of 64 latent channels), four waves: qa[t][h][r] = sum_d q_u[d] W_uk[h * dim + d][r].  Lane = channel r (the
// matrix rows are read coalesced), wave w sums a quarter of the d range, the quarters meet in LDS.  Chunk 0 also copies q_r behind.
__global__ void __launch_bounds__(256) k_latent_absorb_q(const float *__restrict__ q, size_t ldq, int dim, int dr, int R, const bf16_t *__restrict__ wuk,
                                                         float *__restrict__ qa, size_t ldqa)
{
    __shared__ float part[4][64];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *qh = q + (size_t)t * ldq + (size_t)h * (dim + dr);
    float *out = qa + (size_t)t * ldqa + (size_t)h * (R + dr);
    const int r = blockIdx.z * 64 + lane, dq = (dim + 3) / 4, d0 = wave * dq, d1 = min(dim, d0 + dq);
    const bf16_t *w = wuk + (size_t)h * dim * R + r;
    float acc = 0.0f;
    if (r < R) {
#pragma unroll 8
        for (int d = d0; d < d1; d++) acc = fmaf(qh[d], bf2f(w[(size_t)d * R]), acc);
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && r < R) out[r] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
    if (blockIdx.z == 0) for (int e = threadIdx.x; e < dr; e += blockDim.x) out[R + e] = qh[dim + e];
}

// grid (rows, groups of four output columns), a wave per column c = h * vdim + e: out[t][c] = gate[t][h] * sum_r W_uv[c][r] ol[t][h * ld_head + r]
__global__ void __launch_bounds__(256) k_latent_expand_out(const float *__restrict__ ol, size_t ldol, int ld_head, int heads, int vdim, int R, const bf16_t *__restrict__ wuv,
                                                           const float *__restrict__ g, size_t ldg, float *__restrict__ out, size_t ldo, int vec)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63, c = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (c >= heads * vdim) return;
    const int h = c / vdim;
    const float *src = ol + (size_t)t * ldol + (size_t)h * ld_head;
    const bf16_t *w = wuv + (size_t)c * R;
    float acc = 0.0f;
    if (vec) {
        for (int r = lane * 8; r < R; r += 512) {
            const uint4 wv = *reinterpret_cast<const uint4 *>(w + r);
            const float4 a0 = *reinterpret_cast<const float4 *>(src + r), a1 = *reinterpret_cast<const float4 *>(src + r + 4);
            acc = fmaf(a0.x, __uint_as_float(wv.x << 16), acc); acc = fmaf(a0.y, __uint_as_float(wv.x & 0xFFFF0000u), acc);
            acc = fmaf(a0.z, __uint_as_float(wv.y << 16), acc); acc = fmaf(a0.w, __uint_as_float(wv.y & 0xFFFF0000u), acc);
            acc = fmaf(a1.x, __uint_as_float(wv.z << 16), acc); acc = fmaf(a1.y, __uint_as_float(wv.z & 0xFFFF0000u), acc);
            acc = fmaf(a1.z, __uint_as_float(wv.w << 16), acc); acc = fmaf(a1.w, __uint_as_float(wv.w & 0xFFFF0000u), acc);
        }
    } else {
        for (int r = lane; r < R; r += 64) acc = fmaf(bf2f(w[r]), src[r], acc);
    }
    acc = wave_sum(acc);
    if (lane == 0) out[(size_t)t * ldo + c] = g ? acc * sigmoid_f(g[(size_t)t * ldg + h]) : acc;
}

// ---- single tokens, absorbed form: the cache rows are keys (kv_rank + rot_dim) and values (the first kv_rank) of ONE head that all
// query heads share.  grid (rows, groups of HB heads, key shares), four waves: a wave walks chunks of 16 keys, four lanes per key for the
// scores of its HB heads (the key row is read ONCE for all of them, the queries sit in LDS), one value column per lane and CPL columns per
// lane for the weighted sums, online softmax per head; the waves meet in LDS and leave {maximum, sum, weighted values} per share, which
// k_attn_latent_rows_combine merges.  Scores, weights and sums are fp32.
struct LatRowArgs {
    const float *q; size_t ldq;                 // absorbed queries [rows][heads * (R + dr)]
    int heads, R, dr;
    float scale;
    const SeqDesc *seqs; const int *row_seq; float *const *slot_base; size_t cache_off;
    float *ws; int nsplit;                      // [rows][heads][nsplit][R + 2]
    float *out; size_t ldo;                     // [rows][heads * R]
    int vec;
};

template <int HB, int CPL>
__global__ void __launch_bounds__(256) k_attn_latent_rows(LatRowArgs P)
{
    extern __shared__ float sm[];
    const int D = P.R + P.dr, dv = P.R;
    float *qs = sm;                              // [HB][D]
    float *wm = qs + HB * D, *wl = wm + 4 * HB;  // [4][HB] each
    float *wacc = wl + 4 * HB;                   // [4][HB][dv]
    const int t = blockIdx.x, h0 = blockIdx.y * HB, split = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nh = min(HB, P.heads - h0);
    const SeqDesc sd = P.seqs[P.row_seq[t]];
    const int i = sd.pos0 + t - sd.row0, nk = i + 1;
    for (int e = tid; e < HB * D; e += blockDim.x) {
        const int hh = e / D, c = e - hh * D;
        qs[e] = hh < nh ? P.q[(size_t)t * P.ldq + (size_t)(h0 + hh) * D + c] : 0.0f;
    }
    __syncthreads();
    const float *kc = P.slot_base[sd.slot] + P.cache_off;
    float m[HB], l[HB], acc[HB][CPL];
#pragma unroll
    for (int hh = 0; hh < HB; hh++) {
        m[hh] = -INFINITY; l[hh] = 0.0f;
#pragma unroll
        for (int e = 0; e < CPL; e++) acc[hh][e] = 0.0f;
    }
    const int nchunks = (nk + 15) / 16, sub = lane & 3;
    for (int ch = split * 4 + wave; ch < nchunks; ch += 4 * P.nsplit) {
        const int vi = ch * 16 + (lane >> 2);
        const bool valid = vi < nk;
        const float *kr = kc + (size_t)(valid ? vi : i) * D;
        float s[HB];
#pragma unroll
        for (int hh = 0; hh < HB; hh++) s[hh] = 0.0f;
        if (P.vec) {
            for (int c = 4 * sub; c < D; c += 16) {
                const float4 kv = *reinterpret_cast<const float4 *>(kr + c);
#pragma unroll
                for (int hh = 0; hh < HB; hh++) {
                    const float *qq = qs + hh * D + c;
                    s[hh] = fmaf(qq[0], kv.x, s[hh]); s[hh] = fmaf(qq[1], kv.y, s[hh]); s[hh] = fmaf(qq[2], kv.z, s[hh]); s[hh] = fmaf(qq[3], kv.w, s[hh]);
                }
            }
        } else {
            for (int c = sub; c < D; c += 4) {
                const float kv = kr[c];
#pragma unroll
                for (int hh = 0; hh < HB; hh++) s[hh] = fmaf(qs[hh * D + c], kv, s[hh]);
            }
        }
        float p[HB];
#pragma unroll
        for (int hh = 0; hh < HB; hh++) {
            const float sc = valid ? quad_sum(s[hh]) * P.scale : -INFINITY;
            const float m_new = fmaxf(m[hh], wave_max(sc));          // finite: the chunk holds at least one visible key
            p[hh] = valid ? expf(sc - m_new) : 0.0f;
            const float corr = m[hh] == -INFINITY ? 0.0f : expf(m[hh] - m_new);
            l[hh] = l[hh] * corr + wave_sum(sub == 0 ? p[hh] : 0.0f);
#pragma unroll
            for (int e = 0; e < CPL; e++) acc[hh][e] *= corr;
            m[hh] = m_new;
        }
        const int cnt = min(16, nk - ch * 16);
        for (int jj = 0; jj < cnt; jj++) {
            const float *vr = kc + (size_t)(ch * 16 + jj) * D;
            float v[CPL];
#pragma unroll
            for (int e = 0; e < CPL; e++) { const int d = lane + 64 * e; v[e] = d < dv ? vr[d] : 0.0f; }
#pragma unroll
            for (int hh = 0; hh < HB; hh++) {
                const float pj = __shfl(p[hh], 4 * jj, 64);
#pragma unroll
                for (int e = 0; e < CPL; e++) acc[hh][e] = fmaf(pj, v[e], acc[hh][e]);
            }
        }
    }
#pragma unroll
    for (int hh = 0; hh < HB; hh++) {
        if (lane == 0) { wm[wave * HB + hh] = m[hh]; wl[wave * HB + hh] = l[hh]; }
#pragma unroll
        for (int e = 0; e < CPL; e++) { const int d = lane + 64 * e; if (d < dv) wacc[(size_t)(wave * HB + hh) * dv + d] = acc[hh][e]; }
    }
    __syncthreads();
    for (int hh = 0; hh < nh; hh++) {
        float M = -INFINITY;
        for (int w = 0; w < 4; w++) M = fmaxf(M, wm[w * HB + hh]);
        float L = 0.0f, f[4];
        for (int w = 0; w < 4; w++) { f[w] = wm[w * HB + hh] == -INFINITY ? 0.0f : expf(wm[w * HB + hh] - M); L += wl[w * HB + hh] * f[w]; }
        float *dst = P.ws + (((size_t)t * P.heads + h0 + hh) * P.nsplit + split) * (dv + 2);
        if (tid == 0) { dst[0] = M; dst[1] = L; }
        for (int d = tid; d < dv; d += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < 4; w++) o = fmaf(wacc[(size_t)(w * HB + hh) * dv + d], f[w], o);
            dst[2 + d] = o;
        }
    }
}

// grid (rows, heads, chunks of 64 value columns), one wave: lane sp holds share sp's maximum and sum (at most 64 shares) for the scale
// factors; then lane = column, the shares' values read four at a time (independent requests, separate sums)
__global__ void __launch_bounds__(64) k_attn_latent_rows_combine(LatRowArgs P)
{
    const int t = blockIdx.x, h = blockIdx.y, dv = P.R, nsplit = P.nsplit, lane = threadIdx.x;
    const float *src = P.ws + ((size_t)t * P.heads + h) * nsplit * (dv + 2);
    const float m_sp = lane < nsplit ? src[(size_t)lane * (dv + 2)] : -INFINITY, l_sp = lane < nsplit ? src[(size_t)lane * (dv + 2) + 1] : 0.0f;
    const float M = wave_max(m_sp);
    const float f_sp = m_sp == -INFINITY ? 0.0f : expf(m_sp - M);
    const float L = wave_sum(l_sp * f_sp);
    const int d = blockIdx.z * 64 + lane;
    const float *col = src + 2 + min(d, dv - 1);
    float o0 = 0.0f, o1 = 0.0f, o2 = 0.0f, o3 = 0.0f;
    int sp = 0;
    for (; sp + 4 <= nsplit; sp += 4) {
        const float v0 = col[(size_t)sp * (dv + 2)], v1 = col[(size_t)(sp + 1) * (dv + 2)], v2 = col[(size_t)(sp + 2) * (dv + 2)], v3 = col[(size_t)(sp + 3) * (dv + 2)];
        o0 = fmaf(v0, __shfl(f_sp, sp, 64), o0); o1 = fmaf(v1, __shfl(f_sp, sp + 1, 64), o1);
        o2 = fmaf(v2, __shfl(f_sp, sp + 2, 64), o2); o3 = fmaf(v3, __shfl(f_sp, sp + 3, 64), o3);
    }
    for (; sp < nsplit; sp++) o0 = fmaf(col[(size_t)sp * (dv + 2)], __shfl(f_sp, sp, 64), o0);
    if (d < dv) P.out[(size_t)t * P.ldo + (size_t)h * dv + d] = ((o0 + o1) + (o2 + o3)) / L;
}

constexpr int LR_HB = 4, LR_MAX_SPLITS = 64;

size_t latent_rows_smem(int R, int dr) { return ((size_t)LR_HB * (R + dr) + 8 * LR_HB + (size_t)4 * LR_HB * R) * 4; }

// LDS beyond 48 KB has to be granted per kernel; `reserved` remembers the largest grant of this instantiation so that a launch
// inside a captured step does not have to ask (ifa_attention_latent_rows_reserve asks ahead)
template <int CPL>
int reserve_latent_rows(size_t smem)
{
    static size_t reserved = 48 * 1024;
    if (smem <= reserved) return IFA_OK;
    IFA_REQUIRE(smem <= 160 * 1024, "ifa_attention_latent_rows_f32: %zu bytes of LDS", smem);
    IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_attn_latent_rows<LR_HB, CPL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    reserved = smem;
    return IFA_OK;
}

int reserve_latent_rows_for(int R, int dr)
{
    const int cpl = (R + 63) / 64;
    const size_t smem = latent_rows_smem(R, dr);
    if (cpl <= 1) return reserve_latent_rows<1>(smem);
    if (cpl <= 2) return reserve_latent_rows<2>(smem);
    if (cpl <= 4) return reserve_latent_rows<4>(smem);
    if (cpl <= 8) return reserve_latent_rows<8>(smem);
    return reserve_latent_rows<16>(smem);
}

template <int CPL>
void launch_latent_rows(const LatRowArgs &P, unsigned rows, hipStream_t s)
{
    hipLaunchKernelGGL((k_attn_latent_rows<LR_HB, CPL>), dim3(rows, (unsigned)((P.heads + LR_HB - 1) / LR_HB), (unsigned)P.nsplit), dim3(256), latent_rows_smem(P.R, P.dr), s, P);
}

// ---- prompts: 128 queries of one sequence per workgroup, the keys 0 .. last query walked in blocks of 32 staged once per workgroup in
// LDS; each wave owns 32 queries: S = Q K^T and O += P V on the fp32 matrix cores (v_mfma_f32_32x32x2_f32: scores and weights stay
// 32-bit), online softmax per query row, P turned from the accumulator layout into an A operand through LDS.  Key columns beyond
// dim + rot_dim and value columns beyond vdim are zero padding up to 32 NTK / 32 NTV.
typedef float f32x16l __attribute__((ext_vector_type(16)));
constexpr int LT_Q = 128, LT_K = 32;

struct LatTileArgs {
    const float *q; size_t ldq;
    int heads, dim, dr, vdim, R;
    float scale;
    const float *kx; size_t ldkx;
    const float *vx; size_t ldvx;
    const int *ctx0;
    const float *g; size_t ldg;
    const SeqDesc *seqs; int n_seqs;
    float *const *slot_base; size_t cache_off;
    float *out; size_t ldo;
    int vec;
};

__device__ __forceinline__ float lt_half_wave_max(float v)      // over the 32 lanes that share lane >> 5
{
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

template <int NTK, int NTV>
__global__ void __launch_bounds__(256) k_attn_latent_tile(LatTileArgs P)
{
    constexpr int DK = 32 * NTK, DKP = DK + 1, DV = 32 * NTV, DVP = DV + 1;
    extern __shared__ float sm[];
    float *Qs = sm;                          // [128][DKP]
    float *Ks = Qs + LT_Q * DKP;             // [32][DKP]
    float *Vs = Ks + LT_K * DKP;             // [32][DVP]
    float *Ps = Vs + LT_K * DVP;             // [4][32][33]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
    const int h = blockIdx.y, dim = P.dim, dk = P.dim + P.dr, dv = P.vdim;
    int tile = blockIdx.x, sq = 0;
    for (; sq < P.n_seqs; sq++) {
        const int nt = (P.seqs[sq].n + LT_Q - 1) / LT_Q;
        if (tile < nt) break;
        tile -= nt;
    }
    if (sq >= P.n_seqs) return;
    const SeqDesc sd = P.seqs[sq];
    const int r0 = sd.row0 + tile * LT_Q, nq = min(LT_Q, sd.n - tile * LT_Q), p0 = sd.pos0 + tile * LT_Q;
    const float *cache = P.slot_base[sd.slot] + P.cache_off + P.R;              // rotated key part of position j: cache + j (R + dr)
    const size_t crow = (size_t)(P.R + P.dr);
    const float *kx = P.kx + (size_t)P.ctx0[sq] * P.ldkx + (size_t)h * dim, *vx = P.vx + (size_t)P.ctx0[sq] * P.ldvx + (size_t)h * dv;
    for (int e = tid; e < LT_Q * (DK / 4); e += 256) {
        const int row = e / (DK / 4), c4 = (e % (DK / 4)) * 4;
        float v4[4] = {0.f, 0.f, 0.f, 0.f};
        if (row < nq) {
            const float *src = P.q + (size_t)(r0 + row) * P.ldq + (size_t)h * dk + c4;
            if (P.vec && c4 + 4 <= dk) { const float4 t4 = *reinterpret_cast<const float4 *>(src); v4[0] = t4.x; v4[1] = t4.y; v4[2] = t4.z; v4[3] = t4.w; }
            else for (int u = 0; u < 4; u++) if (c4 + u < dk) v4[u] = src[u];
        }
        float *d = Qs + row * DKP + c4;
        d[0] = v4[0]; d[1] = v4[1]; d[2] = v4[2]; d[3] = v4[3];
    }
    const int nq_w = min(32, max(0, nq - 32 * wave));             // queries of this wave
    const int qlo = p0 + 32 * wave, qhi = qlo + nq_w - 1;          // their positions
    const int p_last = p0 + nq - 1, nb = p_last / LT_K + 1;
    f32x16l o[NTV];
    float m[16], l[16];
#pragma unroll
    for (int nt = 0; nt < NTV; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[nt][r] = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) { m[r] = -INFINITY; l[r] = 0.0f; }
    float *Pw = Ps + wave * 32 * 33;
    for (int b = 0; b < nb; b++) {
        const int kb0 = b * LT_K, kc_n = min(LT_K, p_last - kb0 + 1);
        __syncthreads();                 // the previous block's K / V reads are done (and Q is staged)
        for (int e = tid; e < LT_K * (DK / 4); e += 256) {
            const int row = e / (DK / 4), c4 = (e % (DK / 4)) * 4;
            float v4[4] = {0.f, 0.f, 0.f, 0.f};
            if (row < kc_n) {
                const float *su = kx + (size_t)(kb0 + row) * P.ldkx, *sr = cache + (size_t)(kb0 + row) * crow;
                if (P.vec && c4 + 4 <= dk) {
                    const float4 t4 = *reinterpret_cast<const float4 *>(c4 < dim ? su + c4 : sr + (c4 - dim));
                    v4[0] = t4.x; v4[1] = t4.y; v4[2] = t4.z; v4[3] = t4.w;
                } else {
                    for (int u = 0; u < 4; u++) { const int c = c4 + u; if (c < dk) v4[u] = c < dim ? su[c] : sr[c - dim]; }
                }
            }
            float *d = Ks + row * DKP + c4;
            d[0] = v4[0]; d[1] = v4[1]; d[2] = v4[2]; d[3] = v4[3];
        }
        for (int e = tid; e < LT_K * (DV / 4); e += 256) {
            const int row = e / (DV / 4), c4 = (e % (DV / 4)) * 4;
            float v4[4] = {0.f, 0.f, 0.f, 0.f};
            if (row < kc_n) {
                const float *sv = vx + (size_t)(kb0 + row) * P.ldvx + c4;
                if (P.vec && c4 + 4 <= dv) { const float4 t4 = *reinterpret_cast<const float4 *>(sv); v4[0] = t4.x; v4[1] = t4.y; v4[2] = t4.z; v4[3] = t4.w; }
                else for (int u = 0; u < 4; u++) if (c4 + u < dv) v4[u] = sv[u];
            }
            float *d = Vs + row * DVP + c4;
            d[0] = v4[0]; d[1] = v4[1]; d[2] = v4[2]; d[3] = v4[3];
        }
        __syncthreads();
        const bool active = nq_w > 0 && kb0 <= qhi;
        if (active) {
            f32x16l acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0.0f;
            const float *qa = Qs + (32 * wave + i) * DKP + g, *ka = Ks + i * DKP + g;
#pragma unroll 8
            for (int s2 = 0; s2 < DK / 2; s2++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[2 * s2], ka[2 * s2], acc, 0, 0, 0);
            const int j = kb0 + i;
            const bool jin = i < kc_n;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int qq = (r & 3) + 8 * (r >> 2) + 4 * g, iq = qlo + qq;
                const bool vis = jin && qq < nq_w && j <= iq;
                const float sc = vis ? acc[r] * P.scale : -INFINITY;
                const float m_new = fmaxf(m[r], lt_half_wave_max(sc));
                const float pr = vis ? expf(sc - m_new) : 0.0f;
                const float corr = m[r] == -INFINITY ? 1.0f : expf(m[r] - m_new);      // (m_new == -inf only while nothing was visible: sums are 0)
                l[r] = l[r] * corr + pr;
                m[r] = m_new;
#pragma unroll
                for (int nt = 0; nt < NTV; nt++) o[nt][r] *= corr;
                Pw[qq * 33 + i] = pr;
            }
        }
        __syncthreads();                 // P of every wave is in LDS
        if (active) {
            const float *pa = Pw + i * 33 + g;
#pragma unroll
            for (int nt = 0; nt < NTV; nt++) {
                const float *va = Vs + g * DVP + 32 * nt + i;
#pragma unroll 8
                for (int s2 = 0; s2 < LT_K / 2; s2++) o[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[2 * s2], va[2 * s2 * DVP], o[nt], 0, 0, 0);
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int qq = (r & 3) + 8 * (r >> 2) + 4 * g;
        float ls = l[r];
#pragma unroll
        for (int of = 16; of > 0; of >>= 1) ls += __shfl_xor(ls, of, 64);
        if (qq >= nq_w) continue;
        const size_t row = (size_t)(r0 + 32 * wave + qq);
        const float gate = P.g ? sigmoid_f(P.g[row * P.ldg + h]) : 1.0f;
        const float sc = gate / ls;
#pragma unroll
        for (int nt = 0; nt < NTV; nt++) if (32 * nt + i < dv) P.out[row * P.ldo + (size_t)h * dv + 32 * nt + i] = o[nt][r] * sc;
    }
}

template <int NTK, int NTV>
int launch_latent_tile(const LatTileArgs &P, unsigned tiles, hipStream_t s)
{
    const size_t smem = ((size_t)(LT_Q + LT_K) * (32 * NTK + 1) + (size_t)LT_K * (32 * NTV + 1) + 4 * 32 * 33) * 4;
    IFA_REQUIRE(smem <= 160 * 1024, "ifa_attention_latent_tile_f32: head sizes need %zu bytes of LDS", smem);
    IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_attn_latent_tile<NTK, NTV>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL((k_attn_latent_tile<NTK, NTV>), dim3(tiles, (unsigned)P.heads), dim3(256), smem, s, P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

template <int NTK>
int dispatch_latent_tile_v(const LatTileArgs &P, unsigned tiles, int ntv, hipStream_t s)
{
    switch (ntv) {
    case 1: return launch_latent_tile<NTK, 1>(P, tiles, s);
    case 2: return launch_latent_tile<NTK, 2>(P, tiles, s);
    case 3: return launch_latent_tile<NTK, 3>(P, tiles, s);
    case 4: return launch_latent_tile<NTK, 4>(P, tiles, s);
    default: return ifa_fail(IFA_ERR_ARG, "ifa_attention_latent_tile_f32: value size above 128");
    }
}

} // namespace

extern "C" {

int ifa_latent_prepare_f32(const void *kv_f32, size_t ldkv, int kv_rank, int rot_dim, int rot_dims, const void *c_norm_w_bf16, float eps,
                           void *q_f32, size_t ldq, int heads, int dim, const double *freq_f64_dev, float rot_mult, const void *seqs_dev,
                           const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t cache_off, ifa_stream stream)
{
    IFA_REQUIRE(kv_f32 && c_norm_w_bf16 && q_f32 && freq_f64_dev && seqs_dev && row_seq_dev && slot_base_dev, "ifa_latent_prepare_f32: null pointer");
    IFA_REQUIRE(kv_rank > 0 && rot_dim >= 0 && rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0 && heads > 0 && dim >= 0 && rows > 0
                && ldkv >= (size_t)(kv_rank + rot_dim) && ldq >= (size_t)heads * (dim + rot_dim), "ifa_latent_prepare_f32: bad shape");
    hipLaunchKernelGGL(k_latent_prepare, dim3((unsigned)rows), dim3(256), (size_t)std::max(rot_dims, 2) * 4, ifa_s(stream), (const float *)kv_f32, ldkv, kv_rank, rot_dim,
                       rot_dims, (const bf16_t *)c_norm_w_bf16, eps, (float *)q_f32, ldq, heads, dim, freq_f64_dev, rot_mult, (const SeqDesc *)seqs_dev, row_seq_dev,
                       (float *const *)slot_base_dev, cache_off);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_latent_absorb_q_f32(const void *q_f32, size_t ldq, int heads, int dim, int rot_dim, int kv_rank, const void *w_uk_bf16, size_t rows,
                            void *qa_f32, size_t ldqa, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && w_uk_bf16 && qa_f32, "ifa_latent_absorb_q_f32: null pointer");
    IFA_REQUIRE(heads > 0 && heads < 65536 && dim > 0 && dim <= 8192 && rot_dim >= 0 && kv_rank > 0 && rows > 0 && ldq >= (size_t)heads * (dim + rot_dim)
                && ldqa >= (size_t)heads * (kv_rank + rot_dim), "ifa_latent_absorb_q_f32: bad shape");
    IFA_REQUIRE(kv_rank <= 64 * 65535, "ifa_latent_absorb_q_f32: latent of %d channels", kv_rank);
    hipLaunchKernelGGL(k_latent_absorb_q, dim3((unsigned)rows, (unsigned)heads, ifa_cdiv((size_t)kv_rank, 64)), dim3(256), 0, ifa_s(stream), (const float *)q_f32, ldq, dim,
                       rot_dim, kv_rank, (const bf16_t *)w_uk_bf16, (float *)qa_f32, ldqa);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_latent_expand_out_f32(const void *ol_f32, size_t ldol, int ld_head, int heads, int vdim, int kv_rank, const void *w_uv_bf16,
                              const void *g_f32, size_t ldg, size_t rows, void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(ol_f32 && w_uv_bf16 && out_f32, "ifa_latent_expand_out_f32: null pointer");
    IFA_REQUIRE(heads > 0 && heads < 65536 && vdim > 0 && kv_rank > 0 && kv_rank <= 8192 && ld_head >= kv_rank && rows > 0 && ldol >= (size_t)(heads - 1) * ld_head + kv_rank
                && ldo >= (size_t)heads * vdim && (!g_f32 || ldg >= (size_t)heads), "ifa_latent_expand_out_f32: bad shape");
    IFA_REQUIRE((size_t)heads * vdim <= 4 * 65535, "ifa_latent_expand_out_f32: %d x %d output columns", heads, vdim);
    // 16-byte requests: whole 8-element pieces in every matrix row, every head's part of a latent row on a 16-byte boundary
    const int vec = (kv_rank % 8 == 0 && ld_head % 4 == 0 && ldol % 4 == 0 && ((uintptr_t)ol_f32 & 15) == 0 && ((uintptr_t)w_uv_bf16 & 15) == 0) ? 1 : 0;
    hipLaunchKernelGGL(k_latent_expand_out, dim3((unsigned)rows, ifa_cdiv((size_t)heads * vdim, 4)), dim3(256), 0, ifa_s(stream), (const float *)ol_f32, ldol, ld_head,
                       heads, vdim, kv_rank, (const bf16_t *)w_uv_bf16, (const float *)g_f32, ldg, (float *)out_f32, ldo, vec);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_attention_latent_rows_f32(const void *qa_f32, size_t ldqa, int heads, int kv_rank, int rot_dim, float scale, const void *seqs_dev,
                                  const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t cache_off, int max_keys, void *ws_f32,
                                  size_t ws_bytes, void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(qa_f32 && seqs_dev && row_seq_dev && slot_base_dev && ws_f32 && out_f32, "ifa_attention_latent_rows_f32: null pointer");
    IFA_REQUIRE(heads > 0 && heads < 65536 * LR_HB && kv_rank > 0 && kv_rank <= 1024 && rot_dim >= 0 && rows > 0 && rows < 65536 && max_keys >= 1
                && ldqa >= (size_t)heads * (kv_rank + rot_dim) && ldo >= (size_t)heads * kv_rank, "ifa_attention_latent_rows_f32: bad shape");
    LatRowArgs P;
    P.q = (const float *)qa_f32; P.ldq = ldqa; P.heads = heads; P.R = kv_rank; P.dr = rot_dim; P.scale = scale; P.seqs = (const SeqDesc *)seqs_dev;
    P.row_seq = row_seq_dev; P.slot_base = (float *const *)slot_base_dev; P.cache_off = cache_off; P.ws = (float *)ws_f32; P.out = (float *)out_f32; P.ldo = ldo;
    P.vec = ((kv_rank + rot_dim) % 4 == 0 && cache_off % 4 == 0) ? 1 : 0;
    // key shares: 64 keys a share over the longest sequence the cache holds (the same for every step, so that a captured step replays),
    // fewer where many rows already fill the chip or the workspace is small
    int nsplit = std::min(LR_MAX_SPLITS, (max_keys + 63) / 64);
    const size_t groups = (size_t)(heads + LR_HB - 1) / LR_HB;
    while (nsplit > 1 && rows * groups * (size_t)nsplit > 2048) nsplit--;
    while (nsplit > 1 && rows * (size_t)heads * nsplit * ((size_t)kv_rank + 2) * 4 > ws_bytes) nsplit--;
    IFA_REQUIRE(rows * (size_t)heads * nsplit * ((size_t)kv_rank + 2) * 4 <= ws_bytes, "ifa_attention_latent_rows_f32: workspace of %zu bytes is too small", ws_bytes);
    P.nsplit = nsplit;
    hipStream_t s = ifa_s(stream);
    int rc;
    if ((rc = reserve_latent_rows_for(kv_rank, rot_dim))) return rc;
    const int cpl = (kv_rank + 63) / 64;
    if (cpl <= 1) launch_latent_rows<1>(P, (unsigned)rows, s);
    else if (cpl <= 2) launch_latent_rows<2>(P, (unsigned)rows, s);
    else if (cpl <= 4) launch_latent_rows<4>(P, (unsigned)rows, s);
    else if (cpl <= 8) launch_latent_rows<8>(P, (unsigned)rows, s);
    else launch_latent_rows<16>(P, (unsigned)rows, s);
    hipLaunchKernelGGL(k_attn_latent_rows_combine, dim3((unsigned)rows, (unsigned)heads, ifa_cdiv((size_t)kv_rank, 64)), dim3(64), 0, s, P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_attention_latent_rows_reserve(int kv_rank, int rot_dim)
{
    IFA_REQUIRE(kv_rank > 0 && kv_rank <= 1024 && rot_dim >= 0, "ifa_attention_latent_rows_reserve: bad shape");
    return reserve_latent_rows_for(kv_rank, rot_dim);
}

int ifa_attention_latent_tile_f32(const void *q_f32, size_t ldq, int heads, int dim, int rot_dim, int vdim, int kv_rank, float scale,
                                  const void *kx_f32, size_t ldkx, const void *vx_f32, size_t ldvx, const int *ctx0_dev, const void *g_f32, size_t ldg,
                                  const void *seqs_dev, const void *seqs_host, int n_seqs, void *const *slot_base_dev, size_t cache_off,
                                  void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && kx_f32 && vx_f32 && ctx0_dev && seqs_dev && seqs_host && slot_base_dev && out_f32, "ifa_attention_latent_tile_f32: null pointer");
    IFA_REQUIRE(heads > 0 && heads < 65536 && dim > 0 && rot_dim >= 0 && vdim > 0 && kv_rank > 0 && n_seqs > 0 && ldq >= (size_t)heads * (dim + rot_dim)
                && ldkx >= (size_t)heads * dim && ldvx >= (size_t)heads * vdim && ldo >= (size_t)heads * vdim && (!g_f32 || ldg >= (size_t)heads),
                "ifa_attention_latent_tile_f32: bad shape");
    const int ntk = (dim + rot_dim + 31) / 32, ntv = (vdim + 31) / 32;
    IFA_REQUIRE(ifa_attention_latent_tile_fits(dim, rot_dim, vdim), "ifa_attention_latent_tile_f32: heads of %d + %d key and %d value dimensions exceed the tile kernel", dim, rot_dim, vdim);
    LatTileArgs P;
    P.q = (const float *)q_f32; P.ldq = ldq; P.heads = heads; P.dim = dim; P.dr = rot_dim; P.vdim = vdim; P.R = kv_rank; P.scale = scale;
    P.kx = (const float *)kx_f32; P.ldkx = ldkx; P.vx = (const float *)vx_f32; P.ldvx = ldvx; P.ctx0 = ctx0_dev; P.g = (const float *)g_f32; P.ldg = ldg;
    P.seqs = (const SeqDesc *)seqs_dev; P.n_seqs = n_seqs; P.slot_base = (float *const *)slot_base_dev; P.cache_off = cache_off; P.out = (float *)out_f32; P.ldo = ldo;
    // 16-byte requests: every source row and every part of a row starts on a 16-byte boundary
    P.vec = (dim % 4 == 0 && rot_dim % 4 == 0 && vdim % 4 == 0 && kv_rank % 4 == 0 && ldq % 4 == 0 && ldkx % 4 == 0 && ldvx % 4 == 0 && cache_off % 4 == 0
             && ((uintptr_t)q_f32 & 15) == 0 && ((uintptr_t)kx_f32 & 15) == 0 && ((uintptr_t)vx_f32 & 15) == 0) ? 1 : 0;
    const ifa_seq_desc *sh = (const ifa_seq_desc *)seqs_host;
    size_t tiles = 0;
    for (int q = 0; q < n_seqs; q++) tiles += ((size_t)sh[q].n + LT_Q - 1) / LT_Q;
    hipStream_t s = ifa_s(stream);
    switch (ntk) {
    case 1: return dispatch_latent_tile_v<1>(P, (unsigned)tiles, ntv, s);
    case 2: return dispatch_latent_tile_v<2>(P, (unsigned)tiles, ntv, s);
    case 3: return dispatch_latent_tile_v<3>(P, (unsigned)tiles, ntv, s);
    case 4: return dispatch_latent_tile_v<4>(P, (unsigned)tiles, ntv, s);
    case 5: return dispatch_latent_tile_v<5>(P, (unsigned)tiles, ntv, s);
    case 6: return dispatch_latent_tile_v<6>(P, (unsigned)tiles, ntv, s);
    default: return ifa_fail(IFA_ERR_ARG, "ifa_attention_latent_tile_f32: key size above 192");
    }
}

int ifa_attention_latent_tile_fits(int dim, int rot_dim, int vdim)
{
    const int ntk = (dim + rot_dim + 31) / 32, ntv = (vdim + 31) / 32;
    if (ntk < 1 || ntk > 6 || ntv < 1 || ntv > 4) return 0;
    const size_t smem = ((size_t)(LT_Q + LT_K) * (32 * ntk + 1) + (size_t)LT_K * (32 * ntv + 1) + 4 * 32 * 33) * 4;
    return smem <= 160 * 1024 ? 1 : 0;
}

} // extern "C"
