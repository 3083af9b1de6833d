// ifa_attn_window.hip -- softmax attention over a per-sequence key / value cache in 32-bit floats with
//   * a sliding window that keeps the first tokens: query i sees key j iff j <= i and (i - j < window or j < keep_first)
//   * grouped queries (query head h reads key / value head h / (heads / kv_heads))
//   * query and key RMS-normed per head without a weight (the keys when they enter the cache)
//   * score = q.k * scale, optional soft cap (cap * tanh(score / cap)), + a learned bias per (distance bucket, head)
//   * a sink per head: exp(sink) joins the denominator, with no key and no value
// Scores, weights and sums are fp32.  The cache rows are [max_ctx][kv_heads * dim] per (slot, layer): K holds the normed keys,
// V the values; a row is addressed by its true position, so kept first tokens keep their distances.
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
};

constexpr int WA_DPL = 4;         // dim <= 64 * WA_DPL

// grid (rows, heads), four waves: the visible keys (kept first tokens, then the window) are walked in chunks of 64, one
// key per lane for the score, one value column per lane for the weighted sum; chunks go round-robin to the waves, each
// with its own running maximum / sum / accumulator, merged through LDS at the end together with the sink.
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
    const int nchunks = (nk + 63) / 64;
    for (int ch = wave; ch < nchunks; ch += 4) {
        const int vi = ch * 64 + lane;
        const bool valid = vi < nk;
        const int j = valid ? (vi < nkeep ? vi : lo + (vi - nkeep)) : i;
        const float *kr = kc + (size_t)j * kvd;
        float s = 0.0f;
        if ((dim & 3) == 0) {
            for (int c = 0; c < dim; c += 4) {
                const float4 kv = *reinterpret_cast<const float4 *>(kr + c);
                s = fmaf(qn[c], kv.x, s); s = fmaf(qn[c + 1], kv.y, s); s = fmaf(qn[c + 2], kv.z, s); s = fmaf(qn[c + 3], kv.w, s);
            }
        } else {
            for (int c = 0; c < dim; c++) s = fmaf(qn[c], kr[c], s);
        }
        s *= P.scale;
        if (P.softcap > 0.0f) s = P.softcap * tanhf(s / P.softcap);
        if (P.rel) s += bf2f(P.rel[(size_t)P.bucket_of[i - j] * P.heads + h]);
        if (!valid) s = -INFINITY;
        const float m_new = fmaxf(m, wave_max(s));          // finite: the chunk holds at least one visible key
        const float p = valid ? expf(s - m_new) : 0.0f;
        const float corr = m == -INFINITY ? 0.0f : expf(m - m_new);
        l = l * corr + wave_sum(p);
#pragma unroll
        for (int e = 0; e < WA_DPL; e++) acc[e] *= corr;
        m = m_new;
        const int cnt = min(64, nk - ch * 64);
        for (int jj = 0; jj < cnt; jj++) {
            const float pj = __shfl(p, jj, 64);
            const int kj = __shfl(j, jj, 64);
            const float *vr = vc + (size_t)kj * kvd;
#pragma unroll
            for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < dim) acc[e] = fmaf(pj, vr[d], acc[e]); }
        }
    }
    if (lane == 0) { wm[wave] = m; wl[wave] = l; }
#pragma unroll
    for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < dim) wacc[wave * dim + d] = acc[e]; }
    __syncthreads();
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
                             void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && seqs_dev && row_seq_dev && slot_base_dev && out_f32, "ifa_attention_window_f32: null pointer");
    IFA_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && rows > 0 && window >= 1 && keep_first >= 0, "ifa_attention_window_f32: bad shape");
    IFA_REQUIRE(dim <= 64 * WA_DPL, "ifa_attention_window_f32: head size %d above %d", dim, 64 * WA_DPL);
    IFA_REQUIRE(!rel_bf16 || (bucket_of_dev && n_buckets > 0), "ifa_attention_window_f32: a bias table needs its bucket map");
    WinAttnArgs P;
    P.q = (const float *)q_f32; P.ldq = ldq; P.heads = heads; P.kv_heads = kv_heads; P.dim = dim; P.norm_q = norm_q; P.eps = eps; P.scale = scale;
    P.softcap = softcap; P.window = window; P.keep_first = keep_first; P.rel = (const bf16_t *)rel_bf16; P.bucket_of = bucket_of_dev; P.n_buckets = n_buckets;
    P.sink = (const bf16_t *)sink_bf16; P.seqs = (const SeqDesc *)seqs_dev; P.row_seq = row_seq_dev; P.slot_base = (float *const *)slot_base_dev;
    P.k_off = k_off; P.v_off = v_off; P.out = (float *)out_f32; P.ldo = ldo;
    const size_t smem = ((size_t)dim * 5 + 8) * 4;
    hipLaunchKernelGGL(k_attn_window, dim3((unsigned)rows, (unsigned)heads), dim3(256), smem, ifa_s(stream), P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

} // extern "C"
