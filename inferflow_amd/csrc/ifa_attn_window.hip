// ifa_attn_window.hip -- softmax attention over a per-sequence key / value cache in 32-bit floats with
//   * a sliding window that keeps the first tokens: query i sees key j iff j <= i and (i - j < window or j < keep_first)
//   * grouped queries (query head h reads key / value head h / (heads / kv_heads))
//   * query and key RMS-normed per head without a weight (the keys when they enter the cache)
//   * score = q.k * scale, optional soft cap (cap * tanh(score / cap)), + a learned bias per (distance bucket, head)
//   * a sink per head: exp(sink) joins the denominator, with no key and no value
// Scores, weights and sums are fp32.  The cache rows are [max_ctx][kv_heads * dim] (K: the normed keys) and [max_ctx][kv_heads * vdim]
// (V) per (slot, layer); a row is addressed by its true position, so kept first tokens keep their distances.
// The same kernels serve attention with rotated queries and keys (ifa_attention_kv_f32): there the norm (with a weight) and the
// rotation are applied by k_qk_rope_store before the keys enter the cache, the values have a size of their own, the sink has a fixed
// score and the window may be unlimited; a layer may read the cache rows that an earlier layer has written.
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
    int heads, kv_heads, dim, vdim;
    int norm_q; float eps, scale, softcap;
    int window, keep_first;
    const bf16_t *rel; const int *bucket_of; int n_buckets;      // rel [n_buckets][heads]; bucket_of [distance]
    const bf16_t *sink;                                          // [heads] or null
    int sink_fixed; float sink_score;                            // sink_fixed != 0 (and sink null): every head's sink has this score
    const SeqDesc *seqs; const int *row_seq; float *const *slot_base; size_t k_off, v_off;
    float *out; size_t ldo;
    float *ws; int nsplit;           // nsplit > 1: the keys of a (row, head) are shared out to nsplit workgroups; partial results in ws [rows][heads][nsplit][dim + 2]
};

__device__ __forceinline__ bool has_sink(const WinAttnArgs &P) { return P.sink != nullptr || P.sink_fixed != 0; }
__device__ __forceinline__ float sink_of(const WinAttnArgs &P, int h) { return P.sink ? bf2f(P.sink[h]) : (P.sink_fixed ? P.sink_score : -INFINITY); }

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
    float *wacc = wl + 4;                             // [4][vdim]
    __shared__ float red[17];
    const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int dim = P.dim, vdim = P.vdim, g = h / (P.heads / P.kv_heads);
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
    const size_t kvd = (size_t)P.kv_heads * dim, vvd = (size_t)P.kv_heads * vdim;
    const float *kc = P.slot_base[sd.slot] + P.k_off + (size_t)g * dim, *vc = P.slot_base[sd.slot] + P.v_off + (size_t)g * vdim;
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
            const float *vr = vc + (size_t)kj * vvd;
#pragma unroll
            for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < vdim) acc[e] = fmaf(pj, vr[d], acc[e]); }
        }
    }
    if (lane == 0) { wm[wave] = m; wl[wave] = l; }
#pragma unroll
    for (int e = 0; e < WA_DPL; e++) { const int d = lane + 64 * e; if (d < vdim) wacc[wave * vdim + d] = acc[e]; }
    __syncthreads();
    if (nsplit > 1) {      // this workgroup's share: maximum, sum and weighted values relative to that maximum; the sink joins in the combine
        float M = -INFINITY;
        for (int w = 0; w < 4; w++) M = fmaxf(M, wm[w]);
        float L = 0.0f, f[4];
        for (int w = 0; w < 4; w++) { f[w] = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M); L += wl[w] * f[w]; }
        float *dst = P.ws + (((size_t)t * P.heads + h) * nsplit + split) * (vdim + 2);
        if (tid == 0) { dst[0] = M; dst[1] = L; }
        for (int d = tid; d < vdim; d += blockDim.x) {
            float o = 0.0f;
            for (int w = 0; w < 4; w++) o = fmaf(wacc[w * vdim + d], f[w], o);
            dst[2 + d] = o;
        }
        return;
    }
    const float snk = sink_of(P, h);
    float M = snk;
    for (int w = 0; w < 4; w++) M = fmaxf(M, wm[w]);
    float L = has_sink(P) ? expf(snk - M) : 0.0f;
    float f[4];
    for (int w = 0; w < 4; w++) { f[w] = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M); L += wl[w] * f[w]; }
    for (int d = tid; d < vdim; d += blockDim.x) {
        float o = 0.0f;
        for (int w = 0; w < 4; w++) o = fmaf(wacc[w * vdim + d], f[w], o);
        P.out[(size_t)t * P.ldo + (size_t)h * vdim + d] = o / L;
    }
}

// grid (rows, heads), one wave: the shares of a (row, head) and its sink into the output row.  Lane sp holds share sp's maximum and
// sum, so the scale factors come from two wave reductions; the weighted values are then read for all shares at once.
constexpr int WA_MAX_SPLITS = 32;

__global__ void __launch_bounds__(64) k_attn_window_combine(WinAttnArgs P)
{
    const int t = blockIdx.x, h = blockIdx.y, dim = P.vdim, nsplit = P.nsplit, lane = threadIdx.x;      // (dim: columns of a value row)
    const float *src = P.ws + ((size_t)t * P.heads + h) * nsplit * (dim + 2);
    const float snk = sink_of(P, h);
    const float m_sp = lane < nsplit ? src[(size_t)lane * (dim + 2)] : -INFINITY, l_sp = lane < nsplit ? src[(size_t)lane * (dim + 2) + 1] : 0.0f;
    const float M = fmaxf(snk, wave_max(m_sp));
    const float f_sp = m_sp == -INFINITY ? 0.0f : expf(m_sp - M);
    const float L = wave_sum(l_sp * f_sp) + (has_sink(P) ? expf(snk - M) : 0.0f);
    // (every lane walks every group of 64 columns, also where it has no column of its own: the scale factors come from other lanes)
    for (int d0 = 0; d0 < dim; d0 += 64) {
        const int d = d0 + lane;
        float v[WA_MAX_SPLITS];
#pragma unroll
        for (int sp = 0; sp < WA_MAX_SPLITS; sp++) v[sp] = (sp < nsplit && d < dim) ? src[(size_t)sp * (dim + 2) + 2 + d] : 0.0f;
        float o = 0.0f;
#pragma unroll
        for (int sp = 0; sp < WA_MAX_SPLITS; sp++) o = fmaf(v[sp], __shfl(f_sp, sp, 64), o);
        if (d < dim) P.out[(size_t)t * P.ldo + (size_t)h * dim + d] = o / L;
    }
}

// ---- prompts: 128 queries of one sequence per workgroup, the visible keys walked in blocks of 32 that are staged ONCE per workgroup
// in LDS; each wave owns 32 queries, one per lane of each half: S^T = K Q^T and O^T += V^T P^T on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32: scores and weights stay 32-bit).  In the transposed products a lane's accumulators hold 16 keys of ITS
// query, so the online softmax (running maximum, weights, rescaling of O^T) is lane-local but for one exchange between the halves,
// and the weights are the second product's B operand as they lie in the accumulators: no trip through LDS.
typedef float f32x16w __attribute__((ext_vector_type(16)));
constexpr int WT_Q = 128, WT_K = 32;

// Key rows of dim <= 32 NTK and value rows of vdim <= 32 NTV floats; the columns beyond are zero in LDS.
template <int NTK, int NTV>
__global__ void __launch_bounds__(256) k_attn_window_tile(WinAttnArgs P, int n_seqs, int vec)
{
    constexpr int DK = 32 * NTK, DKP = DK + 1, DV = 32 * NTV, DVP = DV + 1;
    extern __shared__ float sm[];
    float *Qs = sm;                          // [128][DKP]
    float *Ks = Qs + WT_Q * DKP;             // [32][DKP]
    float *Vs = Ks + WT_K * DKP;             // [32][DVP]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, i = lane & 31, g = lane >> 5;
    const int h = blockIdx.x, kvh = h / (P.heads / P.kv_heads), dk = P.dim, dv = P.vdim;
    // which sequence and which of its 128-row tiles.  The grid runs over (head, tile) with the head as the fast index and the tiles from
    // the last one down: the tiles with the most key blocks start first, and the query heads of a group, which read the same key and
    // value rows, run side by side.
    int tile = (int)(gridDim.y - 1 - blockIdx.y), sq = 0;
    for (; sq < n_seqs; sq++) {
        const int nt = (P.seqs[sq].n + WT_Q - 1) / WT_Q;
        if (tile < nt) break;
        tile -= nt;
    }
    if (sq >= n_seqs) return;
    const SeqDesc sd = P.seqs[sq];
    const int r0 = sd.row0 + tile * WT_Q, nq = min(WT_Q, sd.n - tile * WT_Q), p0 = sd.pos0 + tile * WT_Q;
    const size_t kvd = (size_t)P.kv_heads * dk, vvd = (size_t)P.kv_heads * dv;
    const float *kc = P.slot_base[sd.slot] + P.k_off + (size_t)kvh * dk, *vc = P.slot_base[sd.slot] + P.v_off + (size_t)kvh * dv;
    // Q rows of this wave, normed, into LDS
    for (int rr = 0; rr < 32; rr++) {
        const int q = 32 * wave + rr;
        float v[NTK > 2 ? 2 : 1];
        float ssum = 0.0f;
#pragma unroll
        for (int e = 0; e < (NTK > 2 ? 2 : 1); e++) {
            const int c = lane + 64 * e;
            v[e] = (q < nq && c < dk) ? P.q[(size_t)(r0 + q) * P.ldq + (size_t)h * dk + c] : 0.0f;
            ssum = fmaf(v[e], v[e], ssum);
        }
        const float rinv = P.norm_q ? 1.0f / sqrtf(wave_sum(ssum) / (float)dk + P.eps) : 1.0f;
#pragma unroll
        for (int e = 0; e < (NTK > 2 ? 2 : 1); e++) { const int c = lane + 64 * e; if (c < DK) Qs[q * DKP + c] = v[e] * rinv; }
    }
    const int nq_w = min(32, max(0, nq - 32 * wave));             // queries of this wave
    const int qlo = p0 + 32 * wave, qhi = qlo + nq_w - 1;          // their positions
    const int lo_min = max(0, p0 - P.window + 1), nkeep = min(P.keep_first, lo_min), p_last = p0 + nq - 1;
    const int nb_keep = (nkeep + WT_K - 1) / WT_K, nb_win = (p_last - lo_min + 1 + WT_K - 1) / WT_K;
    f32x16w o[NTV];
    float m = -INFINITY, l = 0.0f;          // of the lane's query (lane & 31)
#pragma unroll
    for (int nt = 0; nt < NTV; nt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[nt][r] = 0.0f;
    // 16-byte path: a thread stages NTK pieces of the key block and NTV of the value block; the pieces of block b + 1 are asked for
    // before block b is worked on and wait in registers meanwhile, so that the loads run behind the matrix-core work
    float4 kreg[NTK], vreg[NTV];
    auto fetch = [&](int b) {
        const bool kept = b < nb_keep;
        const int kb0 = kept ? b * WT_K : lo_min + (b - nb_keep) * WT_K;
        const int kc_n = kept ? min(WT_K, nkeep - kb0) : min(WT_K, p_last - kb0 + 1);
#pragma unroll
        for (int u = 0; u < NTK; u++) {
            const int e = tid + 256 * u, row = e / (DK / 4), c4 = (e % (DK / 4)) * 4;
            kreg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row < kc_n && c4 < dk) kreg[u] = *reinterpret_cast<const float4 *>(kc + (size_t)(kb0 + row) * kvd + c4);
        }
#pragma unroll
        for (int u = 0; u < NTV; u++) {
            const int e = tid + 256 * u, row = e / (DV / 4), c4 = (e % (DV / 4)) * 4;
            vreg[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (row < kc_n && c4 < dv) vreg[u] = *reinterpret_cast<const float4 *>(vc + (size_t)(kb0 + row) * vvd + c4);
        }
    };
    const int nb_all = nb_keep + nb_win;
    if (vec && nb_all > 0) fetch(0);
    for (int b = 0; b < nb_all; b++) {
        const bool kept = b < nb_keep;
        const int kb0 = kept ? b * WT_K : lo_min + (b - nb_keep) * WT_K;
        const int kc_n = kept ? min(WT_K, nkeep - kb0) : min(WT_K, p_last - kb0 + 1);
        __syncthreads();                 // the previous block's K / V reads are done (and Q is staged)
        if (vec) {
#pragma unroll
            for (int u = 0; u < NTK; u++) {
                const int e = tid + 256 * u, row = e / (DK / 4), c4 = (e % (DK / 4)) * 4;
                float *kd = Ks + row * DKP + c4;
                kd[0] = kreg[u].x; kd[1] = kreg[u].y; kd[2] = kreg[u].z; kd[3] = kreg[u].w;
            }
#pragma unroll
            for (int u = 0; u < NTV; u++) {
                const int e = tid + 256 * u, row = e / (DV / 4), c4 = (e % (DV / 4)) * 4;
                float *vd = Vs + row * DVP + c4;
                vd[0] = vreg[u].x; vd[1] = vreg[u].y; vd[2] = vreg[u].z; vd[3] = vreg[u].w;
            }
            if (b + 1 < nb_all) fetch(b + 1);
        } else {
            for (int e = tid; e < WT_K * DK; e += 256) {
                const int row = e / DK, c = e % DK;
                Ks[row * DKP + c] = (row < kc_n && c < dk) ? kc[(size_t)(kb0 + row) * kvd + c] : 0.0f;
            }
            for (int e = tid; e < WT_K * DV; e += 256) {
                const int row = e / DV, c = e % DV;
                Vs[row * DVP + c] = (row < kc_n && c < dv) ? vc[(size_t)(kb0 + row) * vvd + c] : 0.0f;
            }
        }
        __syncthreads();
        const bool active = nq_w > 0 && kb0 <= qhi && (kept || kb0 + kc_n - 1 >= qlo - P.window + 1 || kb0 < P.keep_first);
        if (active) {
            // S^T = K Q^T: the lane's 16 accumulators are 16 KEYS of ITS query (lane & 31), so the running maximum, the weights and the
            // rescaling stay inside the lane but for one exchange between the two halves of the wave
            f32x16w acc;
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r] = 0.0f;
            const float *qa = Qs + (32 * wave + i) * DKP + g, *ka = Ks + i * DKP + g;
#pragma unroll 8
            for (int s2 = 0; s2 < DK / 2; s2++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka[2 * s2], qa[2 * s2], acc, 0, 0, 0);
            const int iq = qlo + i;
            const bool qin = i < nq_w;
            float mloc = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int kk = (r & 3) + 8 * (r >> 2) + 4 * g, j = kb0 + kk;
                const bool vis = qin && kk < kc_n && j <= iq && (iq - j < P.window || j < P.keep_first);
                float sc = acc[r] * P.scale;
                if (P.softcap > 0.0f) sc = P.softcap * tanhf(sc / P.softcap);
                if (P.rel && vis) sc += bf2f(P.rel[(size_t)P.bucket_of[iq - j] * P.heads + h]);
                sc = vis ? sc : -INFINITY;
                acc[r] = sc;
                mloc = fmaxf(mloc, sc);
            }
            mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
            const float m_new = fmaxf(m, mloc);
            const float corr = m == -INFINITY ? 1.0f : expf(m - m_new);      // (m_new == -inf only while nothing was visible: sums are 0)
            float psum = 0.0f;
#pragma unroll
            for (int r = 0; r < 16; r++) { acc[r] = acc[r] == -INFINITY ? 0.0f : expf(acc[r] - m_new); psum += acc[r]; }
            l = l * corr + psum;             // (the keys of this half of the wave; the halves are added at the end)
            m = m_new;
            // O^T += V^T P^T: the weights are the B operand as they lie in the accumulators (step s2 takes keys (s2 & 3) + 8 (s2 >> 2) + 4 g)
#pragma unroll
            for (int nt = 0; nt < NTV; nt++) {
#pragma unroll
                for (int r = 0; r < 16; r++) o[nt][r] *= corr;
                const float *va = Vs + 4 * g * DVP + 32 * nt + i;
#pragma unroll
                for (int s2 = 0; s2 < 16; s2++)
                    o[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(va[((s2 & 3) + 8 * (s2 >> 2)) * DVP], acc[s2], o[nt], 0, 0, 0);
            }
        }
    }
    // the lane holds value columns 32 nt + (r & 3) + 8 (r >> 2) + 4 g of its query
    const float snk = sink_of(P, h);
    const float ls = l + __shfl_xor(l, 32, 64);
    if (i < nq_w) {
        const float M = fmaxf(m, snk);
        const float f = expf(m - M);
        const float L = ls * f + (has_sink(P) ? expf(snk - M) : 0.0f);
        const float sc = f / L;
        float *dst = P.out + (size_t)(r0 + 32 * wave + i) * P.ldo + (size_t)h * dv;
#pragma unroll
        for (int nt = 0; nt < NTV; nt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int c = 32 * nt + (r & 3) + 8 * (r >> 2) + 4 * g;
                if (c < dv) dst[c] = o[nt][r] * sc;
            }
    }
}

// ---- rotated queries and keys.  One workgroup per row, a wave per head at a time: RMS norm over the head's dim values with a weight
// (norm_w bf16 [dim], null: none), then the first rot_dims dimensions turn in pairs (i, i + rot_dims / 2) by the angle pos * freq[i]
// (formed in double: at position 1000 one fp32 ulp of the angle is already 1e-4); the rest pass unchanged.  Query heads are rewritten in
// place; key heads go into the K rows of the cache, the value heads (as projected) into its V rows.  k null: the row brings no keys
// and values of its own (the layer reads another layer's cache rows).
// VX: the values are treated too (v_norm: each value head divided by its root mean square; v_freq: the head then turns by the row's position over
// all vdim dimensions, pair (m, m + vdim / 2) by pos * v_freq[m]) instead of entering the V rows as projected.
template <int RS_CPL, bool VX>
__global__ void __launch_bounds__(256) k_qk_rope_store(float *__restrict__ q, size_t ldq, int heads, const float *__restrict__ k, size_t ldk,
                                                       const float *__restrict__ v, size_t ldv, int kv_heads, int dim, int vdim,
                                                       const bf16_t *__restrict__ q_norm_w, const bf16_t *__restrict__ k_norm_w, float eps, int rot_dims,
                                                       const double *__restrict__ freq, const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq,
                                                       float *const *__restrict__ slot_base, size_t k_off, size_t v_off, int v_norm,
                                                       const double *__restrict__ v_freq)
{
    extern __shared__ float cs[];          // [rot_dims / 2] cos, [rot_dims / 2] sin; VX: [vdim / 2] cos, [vdim / 2] sin behind them
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = blockDim.x >> 6;
    const SeqDesc sd = seqs[row_seq[t]];
    const int pos = sd.pos0 + t - sd.row0, half = rot_dims / 2;
    // VX: two workgroups per row, blockIdx.y 0 for the queries and keys, 1 for the values (each forms only the angles it needs)
    const bool do_qk = !VX || blockIdx.y == 0, do_v = VX && blockIdx.y == 1;
    if (do_qk)
    for (int i = tid; i < half; i += blockDim.x) {
        const double a = (double)pos * freq[i];
        double sn, cn; sincos(a, &sn, &cn);          // (one argument reduction for both)
        cs[i] = (float)cn; cs[half + i] = (float)sn;
    }
    float *vcs = cs + 2 * half;
    const int vhalf = vdim / 2;
    if (do_v && k && v_freq) {
        for (int i = tid; i < vhalf; i += blockDim.x) {
            const double a = (double)pos * v_freq[i];
            double sn, cn; sincos(a, &sn, &cn);
            vcs[i] = (float)cn; vcs[vhalf + i] = (float)sn;
        }
    }
    __syncthreads();
    const int n_items = do_qk ? heads + (k ? kv_heads : 0) : 0;
    for (int it = wave; it < n_items; it += nw) {
        const bool is_q = it < heads;
        const int hd = is_q ? it : it - heads;
        const float *src = is_q ? q + (size_t)t * ldq + (size_t)hd * dim : k + (size_t)t * ldk + (size_t)hd * dim;
        float *dst = is_q ? q + (size_t)t * ldq + (size_t)hd * dim : slot_base[sd.slot] + k_off + ((size_t)pos * kv_heads + hd) * dim;
        const bf16_t *nw_ = is_q ? q_norm_w : k_norm_w;
        float r = 1.0f;
        if (nw_) {
            float s = 0.0f;
            for (int c = lane; c < dim; c += 64) s = fmaf(src[c], src[c], s);
            r = 1.0f / sqrtf(wave_sum(s) / (float)dim + eps);
        }
        // every lane reads both members of its pairs before anything of the head is written (q is rewritten in place); dim <= 64 RS_CPL
        float val[RS_CPL], oth[RS_CPL];
#pragma unroll
        for (int e = 0; e < RS_CPL; e++) {
            const int c = lane + 64 * e;
            val[e] = oth[e] = 0.0f;
            if (c < dim) {
                val[e] = src[c] * r * (nw_ ? bf2f(nw_[c]) : 1.0f);
                if (c < rot_dims) { const int pc = c < half ? c + half : c - half; oth[e] = src[pc] * r * (nw_ ? bf2f(nw_[pc]) : 1.0f); }
            }
        }
#pragma unroll
        for (int e = 0; e < RS_CPL; e++) {
            const int c = lane + 64 * e;
            if (c >= dim) continue;
            float out = val[e];
            if (c < rot_dims) {
                const int fi = c < half ? c : c - half;
                out = c < half ? val[e] * cs[fi] - oth[e] * cs[half + fi] : val[e] * cs[fi] + oth[e] * cs[half + fi];
            }
            dst[c] = out;
        }
    }
    if (VX) {
        if (!k || !do_v) return;
        // a wave per value head: weightless RMS norm, then the turn by the position (a lane reads both members of a pair from the input row)
        for (int hd = wave; hd < kv_heads; hd += nw) {
            const float *src = v + (size_t)t * ldv + (size_t)hd * vdim;
            float *dst = slot_base[sd.slot] + v_off + ((size_t)pos * kv_heads + hd) * vdim;
            float r = 1.0f;
            if (v_norm) {
                float s = 0.0f;
                for (int c = lane; c < vdim; c += 64) s = fmaf(src[c], src[c], s);
                r = 1.0f / sqrtf(wave_sum(s) / (float)vdim + eps);
            }
            for (int c = lane; c < vdim; c += 64) {
                float out = src[c] * r;
                if (v_freq && c < 2 * vhalf) {
                    const int fi = c < vhalf ? c : c - vhalf;
                    const float oth = src[c < vhalf ? c + vhalf : c - vhalf] * r;
                    out = c < vhalf ? out * vcs[fi] - oth * vcs[vhalf + fi] : out * vcs[fi] + oth * vcs[vhalf + fi];
                }
                dst[c] = out;
            }
        }
        return;
    }
    if (k) {
        float *vd = slot_base[sd.slot] + v_off + (size_t)pos * kv_heads * vdim;
        const float *vs = v + (size_t)t * ldv;
        for (int c = tid; c < kv_heads * vdim; c += blockDim.x) vd[c] = vs[c];
    }
}

// heads of a row turned in place by sign * position over their first rot_dims dimensions, pairs (m, m + rot_dims / 2); a workgroup per row
__global__ void __launch_bounds__(256) k_rotate_heads(float *__restrict__ x, size_t ldx, int heads, int dim, int rot_dims, const double *__restrict__ freq, float sign,
                                                      const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq)
{
    extern __shared__ float cs[];          // [rot_dims / 2] cos, [rot_dims / 2] sin
    const int t = blockIdx.x, tid = threadIdx.x, half = rot_dims / 2;
    const SeqDesc sd = seqs[row_seq[t]];
    const int pos = sd.pos0 + t - sd.row0;
    for (int i = tid; i < half; i += blockDim.x) {
        const double a = (double)sign * (double)pos * freq[i];
        double sn, cn; sincos(a, &sn, &cn);          // (one argument reduction for both)
        cs[i] = (float)cn; cs[half + i] = (float)sn;
    }
    __syncthreads();
    float *xr = x + (size_t)t * ldx;
    for (int e = tid; e < heads * half; e += blockDim.x) {      // a thread owns a pair: both members read before either is written
        const int hd = e / half, i = e % half;
        float *p = xr + (size_t)hd * dim;
        const float u = p[i], w = p[i + half];
        p[i] = u * cs[i] - w * cs[half + i];
        p[i + half] = w * cs[i] + u * cs[half + i];
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

static int attention_launch(const char *who, const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int vdim, int norm_q, float eps, float scale, float softcap,
                            int window, int keep_first, const void *rel_bf16, const int *bucket_of_dev, int n_buckets, const void *sink_bf16, int sink_fixed,
                            float sink_score, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                            void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, int max_keys, void *ws_f32, size_t ws_bytes,
                            ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && seqs_dev && row_seq_dev && slot_base_dev && out_f32, "%s: null pointer", who);
    IFA_REQUIRE(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && rows > 0 && window >= 1 && keep_first >= 0, "%s: bad shape", who);
    IFA_REQUIRE(dim <= 64 * WA_DPL_MAX && vdim <= 64 * WA_DPL_MAX, "%s: head size %d / %d above %d", who, dim, vdim, 64 * WA_DPL_MAX);
    IFA_REQUIRE(ldq >= (size_t)heads * dim && ldo >= (size_t)heads * vdim, "%s: row strides %zu / %zu too small", who, ldq, ldo);
    IFA_REQUIRE(!rel_bf16 || (bucket_of_dev && n_buckets > 0), "%s: a bias table needs its bucket map", who);
    WinAttnArgs P;
    P.q = (const float *)q_f32; P.ldq = ldq; P.heads = heads; P.kv_heads = kv_heads; P.dim = dim; P.vdim = vdim; P.norm_q = norm_q; P.eps = eps; P.scale = scale;
    P.softcap = softcap; P.window = window; P.keep_first = keep_first; P.rel = (const bf16_t *)rel_bf16; P.bucket_of = bucket_of_dev; P.n_buckets = n_buckets;
    P.sink = (const bf16_t *)sink_bf16; P.sink_fixed = sink_fixed; P.sink_score = sink_score;
    P.seqs = (const SeqDesc *)seqs_dev; P.row_seq = row_seq_dev; P.slot_base = (float *const *)slot_base_dev;
    P.k_off = k_off; P.v_off = v_off; P.out = (float *)out_f32; P.ldo = ldo; P.ws = nullptr; P.nsplit = 1;
    // prompts: the tiled matrix-core kernel (heads of up to 128 dimensions, zero-padded to whole 32s); single tokens and other sizes: a workgroup per row
    if (rows >= (size_t)tile_min_rows && n_seqs > 0 && dim <= 128 && vdim <= 128) {
        const ifa_seq_desc *sh = (const ifa_seq_desc *)seqs_host;
        size_t tiles = 0;
        for (int q = 0; q < n_seqs; q++) tiles += ((size_t)sh[q].n + WT_Q - 1) / WT_Q;
        const int NTK = (dim + 31) / 32, NTV = (vdim + 31) / 32;
        const size_t smem_t = ((size_t)(WT_Q + WT_K) * (32 * NTK + 1) + (size_t)WT_K * (32 * NTV + 1)) * 4;
        const int vec = (dim % 4 == 0 && vdim % 4 == 0 && k_off % 4 == 0 && v_off % 4 == 0) ? 1 : 0;      // (arena bases are 256-byte aligned)
        IFA_REQUIRE(tiles < 65536, "%s: %zu query tiles in one step", who, tiles);
        const dim3 grid((unsigned)heads, (unsigned)tiles);
#define IFA_WT(K, V) { IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_attn_window_tile<K, V>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_t)); \
                       hipLaunchKernelGGL((k_attn_window_tile<K, V>), grid, dim3(256), smem_t, ifa_s(stream), P, n_seqs, vec); }
#define IFA_WTV(K) { if (NTV == 1) IFA_WT(K, 1) else if (NTV == 2) IFA_WT(K, 2) else if (NTV == 3) IFA_WT(K, 3) else IFA_WT(K, 4) }
        if (NTK == 1) IFA_WTV(1) else if (NTK == 2) IFA_WTV(2) else if (NTK == 3) IFA_WTV(3) else IFA_WTV(4)
#undef IFA_WTV
#undef IFA_WT
        IFA_LAUNCH_CHECK();
        return IFA_OK;
    }
    const size_t smem = ((size_t)dim + 8 + 4 * (size_t)vdim) * 4;
    // few rows: a (row, head)'s keys are shared out to several workgroups (one workgroup pulls its keys through ONE compute unit)
    int nsplit = 1;
    if (ws_f32 && rows * (size_t)heads <= 512) {
        size_t keys = (size_t)window + (size_t)keep_first;
        if (max_keys > 0) keys = std::min(keys, (size_t)max_keys);
        nsplit = (int)std::min<size_t>(WA_MAX_SPLITS, (keys + 63) / 64);
        while (nsplit > 1 && rows * (size_t)heads * nsplit * ((size_t)vdim + 2) * 4 > ws_bytes) nsplit--;
    }
    P.ws = (float *)ws_f32; P.nsplit = nsplit;
    const dim3 grid_rows((unsigned)rows, (unsigned)heads, (unsigned)nsplit);
    if (vdim <= 64) hipLaunchKernelGGL(k_attn_window<1>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (vdim <= 128) hipLaunchKernelGGL(k_attn_window<2>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (vdim <= 256) hipLaunchKernelGGL(k_attn_window<4>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else if (vdim <= 640) hipLaunchKernelGGL(k_attn_window<10>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    else hipLaunchKernelGGL(k_attn_window<WA_DPL_MAX>, grid_rows, dim3(256), smem, ifa_s(stream), P);
    if (nsplit > 1) hipLaunchKernelGGL(k_attn_window_combine, dim3((unsigned)rows, (unsigned)heads), dim3(64), 0, ifa_s(stream), P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_attention_window_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int norm_q, float eps, float scale, float softcap,
                             int window, int keep_first, const void *rel_bf16, const int *bucket_of_dev, int n_buckets, const void *sink_bf16,
                             const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                             void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, void *ws_f32, size_t ws_bytes, ifa_stream stream)
{
    // (the tiled kernel of this entry keeps to whole 32s: other head sizes take a workgroup per row, as before)
    const int tile_ok = dim % 32 == 0 && k_off % 4 == 0 && v_off % 4 == 0;
    return attention_launch("ifa_attention_window_f32", q_f32, ldq, heads, kv_heads, dim, dim, norm_q, eps, scale, softcap, window, keep_first, rel_bf16, bucket_of_dev,
                            n_buckets, sink_bf16, 0, 0.0f, seqs_dev, row_seq_dev, rows, slot_base_dev, k_off, v_off, out_f32, ldo, seqs_host, tile_ok ? n_seqs : 0,
                            tile_min_rows, 0, ws_f32, ws_bytes, stream);
}

int ifa_attention_kv_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int vdim, float scale, int window, int keep_first, int sink,
                         float sink_score, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off,
                         void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, int max_keys, void *ws_f32, size_t ws_bytes,
                         ifa_stream stream)
{
    const int win = window > 0 ? window : (1 << 30);
    return attention_launch("ifa_attention_kv_f32", q_f32, ldq, heads, kv_heads, dim, vdim, 0, 0.0f, scale, 0.0f, win, keep_first, nullptr, nullptr, 0, nullptr,
                            sink ? 1 : 0, sink_score, seqs_dev, row_seq_dev, rows, slot_base_dev, k_off, v_off, out_f32, ldo, seqs_host, n_seqs, tile_min_rows,
                            max_keys, ws_f32, ws_bytes, stream);
}

int ifa_qk_rope_store_f32(void *q_f32, size_t ldq, int heads, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int vdim,
                          const void *q_norm_w_bf16, const void *k_norm_w_bf16, float eps, int rot_dims, const double *freq_f64_dev, const void *seqs_dev,
                          const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off, size_t v_off, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && seqs_dev && row_seq_dev && slot_base_dev && (!k_f32 || v_f32), "ifa_qk_rope_store_f32: null pointer");
    IFA_REQUIRE(heads > 0 && kv_heads > 0 && dim > 0 && dim <= 1024 && vdim > 0 && rows > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0
                && (rot_dims == 0 || freq_f64_dev), "ifa_qk_rope_store_f32: bad shape (head size %d, %d rotated)", dim, rot_dims);
    IFA_REQUIRE(ldq >= (size_t)heads * dim && (!k_f32 || (ldk >= (size_t)kv_heads * dim && ldv >= (size_t)kv_heads * vdim)), "ifa_qk_rope_store_f32: row strides too small");
#define IFA_RS(N) hipLaunchKernelGGL((k_qk_rope_store<N, false>), dim3((unsigned)rows), dim3(256), (size_t)std::max(rot_dims, 2) * 4, ifa_s(stream), (float *)q_f32, ldq, heads, \
                                     (const float *)k_f32, ldk, (const float *)v_f32, ldv, kv_heads, dim, vdim, (const bf16_t *)q_norm_w_bf16, (const bf16_t *)k_norm_w_bf16, eps, \
                                     rot_dims, freq_f64_dev, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, k_off, v_off, 0, (const double *)nullptr)
    if (dim <= 128) IFA_RS(2); else if (dim <= 256) IFA_RS(4); else IFA_RS(16);
#undef IFA_RS
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_qkv_rope_store_f32(void *q_f32, size_t ldq, int heads, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int kv_heads, int dim, int vdim,
                           const void *q_norm_w_bf16, const void *k_norm_w_bf16, float eps, int rot_dims, const double *freq_f64_dev, int v_norm,
                           const double *v_freq_f64_dev, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off,
                           size_t v_off, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && seqs_dev && row_seq_dev && slot_base_dev && (!k_f32 || v_f32), "ifa_qkv_rope_store_f32: null pointer");
    IFA_REQUIRE(heads > 0 && kv_heads > 0 && dim > 0 && dim <= 1024 && vdim > 0 && vdim <= 4096 && rows > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0
                && (rot_dims == 0 || freq_f64_dev) && (!v_freq_f64_dev || vdim % 2 == 0), "ifa_qkv_rope_store_f32: bad shape (head sizes %d / %d, %d rotated)", dim, vdim, rot_dims);
    IFA_REQUIRE(ldq >= (size_t)heads * dim && (!k_f32 || (ldk >= (size_t)kv_heads * dim && ldv >= (size_t)kv_heads * vdim)), "ifa_qkv_rope_store_f32: row strides too small");
    const size_t smem = ((size_t)std::max(rot_dims, 2) + (size_t)vdim + 2) * 4;
#define IFA_RS(N) hipLaunchKernelGGL((k_qk_rope_store<N, true>), dim3((unsigned)rows, k_f32 ? 2u : 1u), dim3(256), smem, ifa_s(stream), (float *)q_f32, ldq, heads, \
                                     (const float *)k_f32, ldk, (const float *)v_f32, ldv, kv_heads, dim, vdim, (const bf16_t *)q_norm_w_bf16, (const bf16_t *)k_norm_w_bf16, eps, \
                                     rot_dims, freq_f64_dev, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, k_off, v_off, v_norm ? 1 : 0, v_freq_f64_dev)
    if (dim <= 128) IFA_RS(2); else if (dim <= 256) IFA_RS(4); else IFA_RS(16);
#undef IFA_RS
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_rotate_heads_f32(void *x_f32, size_t ldx, int heads, int dim, int rot_dims, const double *freq_f64_dev, float sign, const void *seqs_dev,
                         const int *row_seq_dev, size_t rows, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && seqs_dev && row_seq_dev && (rot_dims == 0 || freq_f64_dev), "ifa_rotate_heads_f32: null pointer");
    IFA_REQUIRE(heads > 0 && dim > 0 && rows > 0 && rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && rot_dims <= 8192 && ldx >= (size_t)heads * dim,
                "ifa_rotate_heads_f32: bad shape (head size %d, %d rotated)", dim, rot_dims);
    if (rot_dims == 0) return IFA_OK;
    hipLaunchKernelGGL(k_rotate_heads, dim3((unsigned)rows), dim3(256), (size_t)rot_dims * 4, ifa_s(stream), (float *)x_f32, ldx, heads, dim, rot_dims, freq_f64_dev, sign,
                       (const SeqDesc *)seqs_dev, row_seq_dev);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_attention_kv_sinks_f32(const void *q_f32, size_t ldq, int heads, int kv_heads, int dim, int vdim, float scale, int window, int keep_first,
                               const void *sink_bf16, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t k_off,
                               size_t v_off, void *out_f32, size_t ldo, const void *seqs_host, int n_seqs, int tile_min_rows, int max_keys, void *ws_f32,
                               size_t ws_bytes, ifa_stream stream)
{
    const int win = window > 0 ? window : (1 << 30);
    return attention_launch("ifa_attention_kv_sinks_f32", q_f32, ldq, heads, kv_heads, dim, vdim, 0, 0.0f, scale, 0.0f, win, keep_first, nullptr, nullptr, 0, sink_bf16,
                            0, 0.0f, seqs_dev, row_seq_dev, rows, slot_base_dev, k_off, v_off, out_f32, ldo, seqs_host, n_seqs, tile_min_rows, max_keys, ws_f32, ws_bytes,
                            stream);
}

} // extern "C"
