// ifa_attn_window.hip -- softmax attention over a per-sequence key / value cache in 32-bit floats with
//   * a sliding window that keeps the first tokens: query i sees key j iff j <= i and (i - j < window or j < keep_first)
//   * grouped queries (query head h reads key / value head h / (heads / kv_heads))
//   * query and key RMS-normed per head without a weight (the keys when they enter the cache)
//   * score = q.k * scale, optional soft cap (cap * tanh(score / cap)), + a learned bias per (distance bucket, head)
//   * a sink per head: exp(sink) joins the denominator, with no key and no value
// Scores, weights and sums are fp32.  The cache rows are [max_ctx][kv_heads * dim] per (slot, layer): K holds the normed keys,
// V the values; a row is addressed by its true position, so kept first tokens keep their distances.
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"

using namespace ifa32;

namespace {

// one workgroup per row: K row = k / sqrt(mean_head(k^2) + eps) (norm_k != 0) or k; V row = v as given
__global__ void __launch_bounds__(256) k_kv_store_f32(const float *__restrict__ k, size_t ldk, const float *__restrict__ v, size_t ldv, int kv_heads, int dim,
                                                      int norm_k, float eps, const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq,
                                                      float *const *__restrict__ slot_base, size_t k_off, size_t v_off)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const SeqDesc sd = seqs[row_seq[t]];
    const size_t pos = (size_t)(sd.pos0 + t - sd.row0), kvd = (size_t)kv_heads * dim;
    float *kc = slot_base[sd.slot] + k_off + pos * kvd, *vc = slot_base[sd.slot] + v_off + pos * kvd;
    for (int g = wave; g < kv_heads; g += nw) {
        const float *kr = k + (size_t)t * ldk + (size_t)g * dim, *vr = v + (size_t)t * ldv + (size_t)g * dim;
        float r = 1.0f;
        if (norm_k) {
            float s = 0.0f;
            for (int c = lane; c < dim; c += 64) s = fmaf(kr[c], kr[c], s);
            r = 1.0f / sqrtf(wave_sum(s) / (float)dim + eps);
        }
        for (int c = lane; c < dim; c += 64) { vc[(size_t)g * dim + c] = vr[c]; kc[(size_t)g * dim + c] = kr[c] * r; }
    }
}

struct WinAttnArgs {
    const float *q; size_t ldq;
    int heads, kv_heads, dim;
    int norm_q; float eps, scale, softcap;
    int window, keep_first;
    const bf16_t *rel; const int *bucket_of; int n_buckets;      // rel [n_buckets][heads]; bucket_of [distance]
    const bf16_t *sink;                                          // [heads] or null
    const SeqDesc *seqs; const int *row_seq; float *const *slot_base; size_t k_off, v_off;
    float *out; size_t ldo;
    float *ws; int nsplit;           // nsplit > 1: the keys of a (row, head) are shared out to nsplit workgroups; partial results in ws [rows][heads][nsplit][dim + 2]
};

constexpr int WA_DPL_MAX = 16;    // dim <= 64 * DPL: a lane holds DPL value columns (1, 2, 4, 10 or 16: up to 1024, the row of a latent-attention cache)

// grid (rows, heads, splits), four waves: the visible keys (kept first tokens, then the window) are walked in chunks of 16, four
// lanes per key for the score, one value column per lane for the weighted sum; chunks go round-robin to the waves, each
// with its own running maximum / sum / accumulator, merged through LDS at the end together with the sink.
template <int WA_DPL>
__global__ void __launch_bounds__(256) k_attn_window(WinAttnArgs P)
{
    extern __shared__ float sm[];
    float *qn = sm;                                   // [dim]
    float *wm = sm + P.dim, *wl = wm + 4;             // per wave: maximum, sum
    float *wacc = wl + 4;                             // [4][dim]
    __shared__ float red[17];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dim = P.dim, g = h / (P.heads / P.kv_heads);
    const SeqDesc sd = P.seqs[P.row_seq[t]];
    const int i = sd.pos0 + t - sd.row0;
    {
        const float *qr = P.q + (size_t)t * P.ldq + (size_t)h * dim;
        float s = 0.0f;
        for (int c = tid; c < dim; c += blockDim.x) s = fmaf(qr[c], qr[c], s);
        const float r = P.norm_q ? 1.0f / sqrtf(block_sum(s, red) / (float)dim + P.eps) : 1.0f;
        for (int c = tid; c < dim; c += blockDim.x) qn[c] = qr[c] * r;
    }
    __syncthreads();
    const int lo = max(0, i - P.window + 1), nkeep = min(P.keep_first, lo), nk = nkeep + (i - lo + 1);
    const size_t kvd = (size_t)P.kv_heads * dim;
    const float *kc = P.slot_base[sd.slot] + P.k_off + (size_t)g * dim, *vc = P.slot_base[sd.slot] + P.v_off + (size_t)g * dim;
    float m = -INFINITY, l = 0.0f, acc[WA_DPL];
#pragma unroll
    for (int e = 0; e < WA_DPL; e++) acc[e] = 0.0f;
    // 16 keys per wave and step, four lanes per key (each a quarter of the dot product in interleaved 16-byte pieces, finished by a quad sum)
    const int nchunks = (nk + 15) / 16, sub = lane & 3;
    const int nsplit = max(1, P.nsplit), split = blockIdx.z;
    for (int ch = split * 4 + wave; ch < nchunks; ch += 4 * nsplit) {
        const int vi = ch * 16 + (lane >> 2);
        const bool valid = vi < nk;
        const int j = valid ? (vi < nkeep ? vi : lo + (vi - nkeep)) : i;
        const float *kr = kc + (size_t)j * kvd;
        float s = 0.0f;
        if ((dim & 3) == 0) {
            for (int c = 4 * sub; c < dim; c += 16) {
                const float4 kv = *reinterpret_cast<const float4 *>(kr + c);
                s = fmaf(qn[c], kv.x, s); s = fmaf(qn[c + 1], kv.y, s); s = fmaf(qn[c + 2], kv.z, s); s = fmaf(qn[c + 3], kv.w, s);
            }
        } else {
            for (int c = sub; c < dim; c += 4) s = fmaf(qn[c], kr[c], s);
        }
        s = quad_sum(s) * P.scale;
        if (P.softcap > 0.0f) s = P.softcap * tanhf(s / P.softcap);
        if (P.rel) s += bf2f(P.rel[(size_t)P.bucket_of[i - j] * P.heads + h]);
        if (!valid) s = -INFINITY;
        const float m_new = fmaxf(m, wave_max(s));          // finite: the chunk holds at least one visible key
        const float p = valid ? expf(s - m_new) : 0.0f;
        const float corr = m == -INFINITY ? 0.0f : expf(m - m_new);
        l = l * corr + wave_sum(sub == 0 ? p : 0.0f);
#pragma unroll
        for (int e = 0; e < WA_DPL; e++) acc[e] *= corr;
        m = m_new;
        const int cnt = min(16, nk - ch * 16);
        for (int jj = 0; jj < cnt; jj++) {
            const float pj = __shfl(p, 4 * jj, 64);
            const int kj = __shfl(j, 4 * jj, 64);
            const float *vr = vc + (size_t)kj * kvd;
#pragma unroll
            for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < dim) acc[e] = fmaf(pj, vr[d], acc[e]); }
        }
    }
    if (lane == 0) { wm[wave] = m; wl[wave] = l; }
#pragma unroll
    for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < dim) wacc[wave * dim + d] = acc[e]; }
    __syncthreads();
    if (nsplit > 1) {      // this workgroup's share: maximum, sum and weighted values relative to that maximum; the sink joins in the combine
        float M = -INFINITY;
        for (int w = 0; w < 4; w++) M = fmaxf(M, wm[w]);
        float L = 0.0f, f[4];
        for (int w = 0; w < 4; w++) { f[w] = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M); L += wl[w] * f[w]; }
        float *dst = P.ws + (((size_t)t * P.heads + h) * nsplit + split) * (dim + 2);
        if (tid == 0) { dst[0] = M; dst[1] = L; }
        for (int d = tid; d < dim; d += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < 4; w++) o = fmaf(wacc[w * dim + d], f[w], o);
            dst[2 + d] = o;
        }
        return;
    }
    const float snk = P.sink ? bf2f(P.sink[h]) : -INFINITY;
    float M = snk;
    for (int w = 0; w < 4; w++) M = fmaxf(M, wm[w]);
    float L = P.sink ? expf(snk - M) : 0.0f;
    float f[4];
    for (int w = 0; w < 4; w++) { f[w] = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M); L += wl[w] * f[w]; }
    for (int d = tid; d < dim; d += blockDim.x) {
        float o = 0.0f;
        for (int w = 0; w < 4; w++) o = fmaf(wacc[w * dim + d], f[w], o);
        P.out[(size_t)t * P.ldo + (size_t)h * dim + d] = o / L;
    }
}

// grid (rows, heads), one wave: the shares of a (row, head) and its sink into the output row.  Lane sp holds share sp's maximum and
// sum, so the scale factors come from two wave reductions; the weighted values are then read for all shares at once.
constexpr int WA_MAX_SPLITS = 32;

__global__ void __launch_bounds__(64) k_attn_window_combine(WinAttnArgs P)
{
    const int t = blockIdx.x, h = blockIdx.y, dim = P.dim, nsplit = P.nsplit, lane = threadIdx.x;
    const float *src = P.ws + ((size_t)t * P.heads + h) * nsplit * (dim + 2);
    const float snk = P.sink ? bf2f(P.sink[h]) : -INFINITY;
    const float m_sp = lane < nsplit ? src[(size_t)lane * (dim + 2)] : -INFINITY, l_sp = lane < nsplit ? src[(size_t)lane * (dim + 2) + 1] : 0.0f;
    const float M = fmaxf(snk, wave_max(m_sp));
    const float f_sp = m_sp == -INFINITY ? 0.0f : expf(m_sp - M);
    const float L = wave_sum(l_sp * f_sp) + (P.sink ? expf(snk - M) : 0.0f);
    for (int d = lane; d < dim; d += 64) {
        float v[WA_MAX_SPLITS];
#pragma unroll
        for (int sp = 0; sp < WA_MAX_SPLITS; sp++) v[sp] = sp < nsplit ? src[(size_t)sp * (dim + 2) + 2 + d] : 0.0f;
        float o = 0.0f;
#pragma unroll
        for (int sp = 0; sp < WA_MAX_SPLITS; sp++) o = fmaf(v[sp], __shfl(f_sp, sp, 64), o);
        P.out[(size_t)t * P.ldo + (size_t)h * dim + d] = o / L;
    }
}

// ---- prompts: 128 queries of one sequence per workgroup, the visible keys walked in blocks of 32 that are staged ONCE per workgroup
// in LDS; each wave owns 32 queries: S = Q K^T and O += P V on the fp32 matrix cores (v_mfma_f32_32x32x2_f32: scores and weights
// stay 32-bit), online softmax per query row (running maximum across the block's keys by lane exchange, the row sums kept per lane
// and added up once at the end), P turned from the accumulator layout into an A operand through LDS.  dim = 32 NT.
typedef float f32x16w __attribute__((ext_vector_type(16)));
constexpr int WT_Q = 128, WT_K = 32;

__device__ __forceinline__ float half_wave_max(float v)      // over the 32 lanes that share lane >> 5
{
#pragma unroll
    for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

template <int NT>
__global__ void __launch_bounds__(256) k_attn_window_tile(WinAttnArgs P, int n_seqs)
{
    constexpr int D = 32 * NT, DP = D + 1;
    extern __shared__ float sm[];
    float *Qs = sm;                          // [128][DP]
    float *Ks = Qs + WT_Q * DP;              // [32][DP]
    float *Vs = Ks + WT_K * DP;              // [32][DP]
    float *Ps = Vs + WT_K * DP;              // [4][32][33]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
    const int h = blockIdx.y, kvh = h / (P.heads / P.kv_heads);
    // which sequence and which of its 128-row tiles
    int tile = blockIdx.x, sq = 0;
    for (; sq < n_seqs; sq++) {
        const int nt = (P.seqs[sq].n + WT_Q - 1) / WT_Q;
        if (tile < nt) break;
        tile -= nt;
    }
    if (sq >= n_seqs) return;
    const SeqDesc sd = P.seqs[sq];
    const int r0 = sd.row0 + tile * WT_Q, nq = min(WT_Q, sd.n - tile * WT_Q), p0 = sd.pos0 + tile * WT_Q;
    const size_t kvd = (size_t)P.kv_heads * D;
    const float *kc = P.slot_base[sd.slot] + P.k_off + (size_t)kvh * D, *vc = P.slot_base[sd.slot] + P.v_off + (size_t)kvh * D;
    // Q rows of this wave, normed, into LDS
    for (int rr = 0; rr < 32; rr++) {
        const int q = 32 * wave + rr;
        float v[NT > 2 ? 2 : 1];
        float ssum = 0.0f;
#pragma unroll
        for (int e = 0; e < (NT > 2 ? 2 : 1); e++) {
            const int c = lane + 64 * e;
            v[e] = (q < nq && c < D) ? P.q[(size_t)(r0 + q) * P.ldq + (size_t)h * D + c] : 0.0f;
            ssum = fmaf(v[e], v[e], ssum);
        }
        const float rinv = P.norm_q ? 1.0f / sqrtf(wave_sum(ssum) / (float)D + P.eps) : 1.0f;
#pragma unroll
        for (int e = 0; e < (NT > 2 ? 2 : 1); e++) { const int c = lane + 64 * e; if (c < D) Qs[q * DP + c] = v[e] * rinv; }
    }
    const int nq_w = min(32, max(0, nq - 32 * wave));             // queries of this wave
    const int qlo = p0 + 32 * wave, qhi = qlo + nq_w - 1;          // their positions
    const int lo_min = max(0, p0 - P.window + 1), nkeep = min(P.keep_first, lo_min), p_last = p0 + nq - 1;
    const int nb_keep = (nkeep + WT_K - 1) / WT_K, nb_win = (p_last - lo_min + 1 + WT_K - 1) / WT_K;
    f32x16w o[NT];
    float m[16], l[16];
#pragma unroll
    for (int nt = 0; nt < NT; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[nt][r] = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r++) { m[r] = -INFINITY; l[r] = 0.0f; }
    float *Pw = Ps + wave * 32 * 33;
    for (int b = 0; b < nb_keep + nb_win; b++) {
        const bool kept = b < nb_keep;
        const int kb0 = kept ? b * WT_K : lo_min + (b - nb_keep) * WT_K;
        const int kc_n = kept ? min(WT_K, nkeep - kb0) : min(WT_K, p_last - kb0 + 1);
        __syncthreads();                 // the previous block's K / V reads are done (and Q is staged)
        for (int e = tid; e < WT_K * (D / 4); e += 256) {
            const int row = e / (D / 4), c4 = (e % (D / 4)) * 4;
            float4 kv = make_float4(0.f, 0.f, 0.f, 0.f), vv = kv;
            if (row < kc_n) {
                kv = *reinterpret_cast<const float4 *>(kc + (size_t)(kb0 + row) * kvd + c4);
                vv = *reinterpret_cast<const float4 *>(vc + (size_t)(kb0 + row) * kvd + c4);
            }
            float *kd = Ks + row * DP + c4, *vd = Vs + row * DP + c4;
            kd[0] = kv.x; kd[1] = kv.y; kd[2] = kv.z; kd[3] = kv.w;
            vd[0] = vv.x; vd[1] = vv.y; vd[2] = vv.z; vd[3] = vv.w;
        }
        __syncthreads();
        const bool active = nq_w > 0 && kb0 <= qhi && (kept || kb0 + kc_n - 1 >= qlo - P.window + 1 || kb0 < P.keep_first);
        if (active) {
            f32x16w acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0.0f;
            const float *qa = Qs + (32 * wave + i) * DP + g, *ka = Ks + i * DP + g;
#pragma unroll 8
            for (int s2 = 0; s2 < D / 2; s2++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa[2 * s2], ka[2 * s2], acc, 0, 0, 0);
            const int j = kb0 + i;
            const bool jin = i < kc_n;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int q = (r & 3) + 8 * (r >> 2) + 4 * g, iq = qlo + q;
                const bool vis = jin && q < nq_w && j <= iq && (iq - j < P.window || j < P.keep_first);
                float sc = acc[r] * P.scale;
                if (P.softcap > 0.0f) sc = P.softcap * tanhf(sc / P.softcap);
                if (P.rel && vis) sc += bf2f(P.rel[(size_t)P.bucket_of[iq - j] * P.heads + h]);
                sc = vis ? sc : -INFINITY;
                const float m_new = fmaxf(m[r], half_wave_max(sc));
                const float pr = vis ? expf(sc - m_new) : 0.0f;
                const float corr = m[r] == -INFINITY ? 1.0f : expf(m[r] - m_new);      // (m_new == -inf only while nothing was visible: sums are 0)
                l[r] = l[r] * corr + pr;
                m[r] = m_new;
#pragma unroll
                for (int nt = 0; nt < NT; nt++) o[nt][r] *= corr;
                Pw[q * 33 + i] = pr;
            }
        }
        __syncthreads();                 // P of every wave is in LDS
        if (active) {
            const float *pa = Pw + i * 33 + g;
#pragma unroll
            for (int nt = 0; nt < NT; nt++) {
                const float *va = Vs + g * DP + 32 * nt + i;
#pragma unroll 8
                for (int s2 = 0; s2 < WT_K / 2; s2++) o[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(pa[2 * s2], va[2 * s2 * DP], o[nt], 0, 0, 0);
            }
        }
    }
    const float snk = P.sink ? bf2f(P.sink[h]) : -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int q = (r & 3) + 8 * (r >> 2) + 4 * g;
        float ls = l[r];
#pragma unroll
        for (int of = 16; of > 0; of >>= 1) ls += __shfl_xor(ls, of, 64);
        if (q >= nq_w) continue;
        const float M = fmaxf(m[r], snk);
        const float f = expf(m[r] - M);
        const float L = ls * f + (P.sink ? expf(snk - M) : 0.0f);
        const float sc = f / L;
#pragma unroll
        for (int nt = 0; nt < NT; nt++) P.out[(size_t)(r0 + 32 * wave + q) * P.ldo + (size_t)h * D + 32 * nt + i] = o[nt][r] * sc;
    }
}

} // namespace

extern "C" {

int ifa_kv_store_f32(const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int norm_k, float eps, const void *seqs_dev,
                     const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off, ifa_stream stream)
{
    IFA_REQUIRE(k_f32 && v_f32 && seqs_dev && row_seq_dev && slot_base_dev, "ifa_kv_store_f32: null pointer");
    IFA_REQUIRE(kv_heads > 0 && dim > 0 && rows > 0 && ldk >= (size_t)kv_heads * dim && ldv >= (size_t)kv_heads * dim, "ifa_kv_store_f32: bad shape");
    hipLaunchKernelGGL(k_kv_store_f32, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const float *)k_f32, ldk, (const float *)v_f32, ldv, kv_heads, dim,
                       norm_k, eps, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, k_off, v_off);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_attention_window_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int norm_q, float eps, float scale, float softcap,
                             int window, int keep_first, const void *rel_bf16, const int *bucket_of_dev, int n_buckets, const void *sink_bf16,
                             const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                             void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, void *ws_f32, size_t ws_bytes, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && seqs_dev && row_seq_dev && slot_base_dev && out_f32, "ifa_attention_window_f32: null pointer");
    IFA_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && rows > 0 && window >= 1 && keep_first >= 0, "ifa_attention_window_f32: bad shape");
    IFA_REQUIRE(dim <= 64 * WA_DPL_MAX, "ifa_attention_window_f32: head size %d above %d", dim, 64 * WA_DPL_MAX);
    IFA_REQUIRE(!rel_bf16 || (bucket_of_dev && n_buckets > 0), "ifa_attention_window_f32: a bias table needs its bucket map");
    WinAttnArgs P;
    P.q = (const float *)q_f32; P.ldq = ldq; P.heads = heads; P.kv_heads = kv_heads; P.dim = dim; P.norm_q = norm_q; P.eps = eps; P.scale = scale;
    P.softcap = softcap; P.window = window; P.keep_first = keep_first; P.rel = (const bf16_t *)rel_bf16; P.bucket_of = bucket_of_dev; P.n_buckets = n_buckets;
    P.sink = (const bf16_t *)sink_bf16; P.seqs = (const SeqDesc *)seqs_dev; P.row_seq = row_seq_dev; P.slot_base = (float *const *)slot_base_dev;
    P.k_off = k_off; P.v_off = v_off; P.out = (float *)out_f32; P.ldo = ldo; P.ws = nullptr; P.nsplit = 1;
    // prompts: the tiled matrix-core kernel (head sizes 32 / 64 / 96 / 128, 16-byte aligned cache rows); single tokens and other sizes: a workgroup per row
    if (rows >= (size_t)tile_min_rows && n_seqs > 0 && dim % 32 == 0 && dim <= 128 && k_off % 4 == 0 && v_off % 4 == 0) {
        const ifa_seq_desc *sh = (const ifa_seq_desc *)seqs_host;
        size_t tiles = 0;
        for (int q = 0; q < n_seqs; q++) tiles += ((size_t)sh[q].n + WT_Q - 1) / WT_Q;
        const int NT = dim / 32, DP = dim + 1;
        const size_t smem_t = ((size_t)(WT_Q + 2 * WT_K) * DP + 4 * 32 * 33) * 4;
        const dim3 grid((unsigned)tiles, (unsigned)heads);
#define IFA_WT(N) { IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_attn_window_tile<N>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_t)); \
                    hipLaunchKernelGGL(k_attn_window_tile<N>, grid, dim3(256), smem_t, ifa_s(stream), P, n_seqs); }
        if (NT == 1) IFA_WT(1) else if (NT == 2) IFA_WT(2) else if (NT == 3) IFA_WT(3) else IFA_WT(4)
#undef IFA_WT
        IFA_LAUNCH_CHECK();
        return IFA_OK;
    }
    const size_t smem = ((size_t)dim * 5 + 8) * 4;
    // few rows: a (row, head)'s keys are shared out to several workgroups (one workgroup pulls its keys through ONE compute unit)
    int nsplit = 1;
    if (ws_f32 && rows * (size_t)heads <= 512) {
        nsplit = (int)std::min<size_t>(WA_MAX_SPLITS, ((size_t)window + (size_t)keep_first + 63) / 64);
        while (nsplit > 1 && rows * (size_t)heads * nsplit * ((size_t)dim + 2) * 4 > ws_bytes) nsplit--;
    }
    P.ws = (float *)ws_f32; P.nsplit = nsplit;
    const dim3 grid_rows((unsigned)rows, (unsigned)heads, (unsigned)nsplit);
    if (dim <= 64) hipLaunchKernelGGL(k_attn_window<1>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (dim <= 128) hipLaunchKernelGGL(k_attn_window<2>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (dim <= 256) hipLaunchKernelGGL(k_attn_window<4>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (dim <= 640) hipLaunchKernelGGL(k_attn_window<10>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else hipLaunchKernelGGL(k_attn_window<WA_DPL_MAX>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    if (nsplit > 1) hipLaunchKernelGGL(k_attn_window_combine, dim3((unsigned)rows, (unsigned)heads), dim3(64), 0, ifa_s(stream), P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

} // extern "C"
