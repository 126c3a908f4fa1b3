// ifa_moe_f32.hip -- mixture of experts on 32-bit activations with bfloat16 expert matrices:
//   router   scores = softmax(logits) over `experts` feed-forward experts followed by `identity` identity experts; the `top` largest
//            (score + correction) are chosen, their weights are the plain scores (not renormalized)
//            (second kind, k_moe_route_top: the `top` largest logit + bias, weights = softmax over the chosen values only)
//   experts  y[t] (+)= sum_k wgt[t][k] * E_{idx[t][k]}(h[t]),  E_e(h) = W_down[e] act(W_up[e] h),  identity: E(h) = h
//            (gated experts: E_e(h) = W_down[e] (silu(W_gate[e] h) * (W_up[e] h)), gate and up rows of an expert stored back to back)
// Few rows (decode steps): every (row, choice) pair streams its expert's matrices, a wave per output (k_moe_up_rows / k_moe_down_rows).
// Many rows: the pairs are sorted by expert (k_moe_sort: counts, offsets and tiles of 64 rows of one expert, all in one workgroup),
// both products run grouped on the matrix cores (ifa_linear_bf16w_grouped: gather of the rows in the first, activation in its epilogue,
// the pair's weight in the second's) and k_moe_combine adds a row's pairs in the fixed order of its choices.  No atomics on values: a
// row's result does not depend on what else is in the step.
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"
#include "inferflow_amd.h"

using namespace ifa32;

namespace {

typedef uint32_t u32x4m __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float gelu_erf_f(float z) { return 0.5f * z * (1.0f + erff(z * 0.70710678118654752f)); }

// one wave per row: softmax over n_all logits, then `top` passes of argmax over score + correction (lowest index on ties)
// (score_kind 1: the scores are the sigmoids of the logits instead of their softmax)
__global__ void __launch_bounds__(64) k_moe_route(const float *__restrict__ logits, size_t ld, int n_all, int top, const bf16_t *__restrict__ corr,
                                                  int *__restrict__ idx, float *__restrict__ wgt, int score_kind)
{
    extern __shared__ float sc[];          // [n_all] scores, [n_all] choice scores
    float *ch = sc + n_all;
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *z = logits + (size_t)t * ld;
    if (score_kind == 1) {
        for (int e = lane; e < n_all; e += 64) { const float s = sigmoid_f(z[e]); sc[e] = s; ch[e] = s + (corr ? bf2f(corr[e]) : 0.0f); }
    } else {
        float mx = -INFINITY;
        for (int e = lane; e < n_all; e += 64) mx = fmaxf(mx, z[e]);
        mx = wave_max(mx);
        float sum = 0.0f;
        for (int e = lane; e < n_all; e += 64) { const float p = expf(z[e] - mx); sc[e] = p; sum += p; }
        sum = wave_sum(sum);
        for (int e = lane; e < n_all; e += 64) { const float s = sc[e] / sum; sc[e] = s; ch[e] = s + (corr ? bf2f(corr[e]) : 0.0f); }
    }
    __syncthreads();
    for (int k = 0; k < top; k++) {
        float best = -INFINITY; int bi = 0x7FFFFFFF;
        for (int e = lane; e < n_all; e += 64) { const float v = ch[e]; if (v > best || (v == best && e < bi)) { best = v; bi = e; } }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
        }
        if (lane == 0) { idx[(size_t)t * top + k] = bi; wgt[(size_t)t * top + k] = sc[bi]; ch[bi] = -INFINITY; }
        __syncthreads();
    }
}

// one wave per row: `top` passes of argmax over logit + bias (lowest index on ties), then the softmax over the chosen values
__global__ void __launch_bounds__(64) k_moe_route_top(const float *__restrict__ logits, size_t ld, int n_all, int top, const bf16_t *__restrict__ bias,
                                                      int *__restrict__ idx, float *__restrict__ wgt)
{
    extern __shared__ float ch[];          // [n_all] choice values, [top] weights before the division
    float *pw = ch + n_all;
    const int t = blockIdx.x, lane = threadIdx.x;
    const float *z = logits + (size_t)t * ld;
    for (int e = lane; e < n_all; e += 64) ch[e] = z[e] + (bias ? bf2f(bias[e]) : 0.0f);
    __syncthreads();
    float first = 0.0f, sum = 0.0f;
    for (int k = 0; k < top; k++) {
        float best = -INFINITY; int bi = 0x7FFFFFFF;
        for (int e = lane; e < n_all; e += 64) { const float v = ch[e]; if (v > best || (v == best && e < bi)) { best = v; bi = e; } }
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
            if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
        }
        if (k == 0) first = best;                      // the largest of all: the softmax's reference
        const float p = expf(best - first);
        sum += p;
        if (lane == 0) { idx[(size_t)t * top + k] = bi; pw[k] = p; ch[bi] = -INFINITY; }
        __syncthreads();
    }
    for (int k = lane; k < top; k += 64) wgt[(size_t)t * top + k] = pw[k] / sum;
}

// Steps of a few rows: the router's product and its choice in one launch.  A workgroup per row: the waves share out the router's outputs
// (a dot of `width` each), then the scores and the `top` passes as in k_moe_route (wave 0; the other waves only keep the barriers).
// (x not null: the row the router reads is formed here first, h[t] = tanh(alpha x[t]) nw + nb, and written for the experts behind)
__global__ void __launch_bounds__(1024) k_moe_route_rows(const float *h, size_t ldh, int W, const bf16_t *__restrict__ router, int n_all, int top,
                                                        const bf16_t *__restrict__ corr, int *__restrict__ idx, float *__restrict__ wgt, int vec, int score_kind,
                                                        const float *__restrict__ x, size_t ldx, const bf16_t *__restrict__ alpha, const bf16_t *__restrict__ nw_,
                                                        const bf16_t *__restrict__ nb_, float *h_out)
{
    extern __shared__ float sc[];          // [n_all] logits, then scores; [n_all] choice scores
    float *ch = sc + n_all;
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float *hr = h + (size_t)t * ldh;
    if (x) {
        const float a = bf2f(alpha[0]);
        for (int c = threadIdx.x; c < W; c += blockDim.x) h_out[(size_t)t * ldh + c] = fmaf(tanhf(a * x[(size_t)t * ldx + c]), bf2f(nw_[c]), bf2f(nb_[c]));
        __syncthreads();          // (the workgroup reads back what it has written itself)
    }
    for (int e = wave; e < n_all; e += nw) {
        const bf16_t *w = router + (size_t)e * W;
        float acc = 0.0f;
        if (vec) {
#pragma unroll 4
            for (int k = lane * 8; k < W; k += 512) {
                const u32x4m wv = *reinterpret_cast<const u32x4m *>(w + k);
                const float4 a0 = *reinterpret_cast<const float4 *>(hr + k), a1 = *reinterpret_cast<const float4 *>(hr + k + 4);
                acc = fmaf(a0.x, __uint_as_float(wv[0] << 16), acc); acc = fmaf(a0.y, __uint_as_float(wv[0] & 0xFFFF0000u), acc);
                acc = fmaf(a0.z, __uint_as_float(wv[1] << 16), acc); acc = fmaf(a0.w, __uint_as_float(wv[1] & 0xFFFF0000u), acc);
                acc = fmaf(a1.x, __uint_as_float(wv[2] << 16), acc); acc = fmaf(a1.y, __uint_as_float(wv[2] & 0xFFFF0000u), acc);
                acc = fmaf(a1.z, __uint_as_float(wv[3] << 16), acc); acc = fmaf(a1.w, __uint_as_float(wv[3] & 0xFFFF0000u), acc);
            }
        } else {
            for (int k = lane; k < W; k += 64) acc = fmaf(hr[k], bf2f(w[k]), acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) sc[e] = acc;
    }
    __syncthreads();
    if (wave == 0 && score_kind == 1) {
        for (int e = lane; e < n_all; e += 64) { const float sv = sigmoid_f(sc[e]); sc[e] = sv; ch[e] = sv + (corr ? bf2f(corr[e]) : 0.0f); }
    } else if (wave == 0) {
        float mx = -INFINITY;
        for (int e = lane; e < n_all; e += 64) mx = fmaxf(mx, sc[e]);
        mx = wave_max(mx);
        float sum = 0.0f;
        for (int e = lane; e < n_all; e += 64) { const float pe = expf(sc[e] - mx); sc[e] = pe; sum += pe; }      // (each lane touches its own entries only)
        sum = wave_sum(sum);
        for (int e = lane; e < n_all; e += 64) { const float sv = sc[e] / sum; sc[e] = sv; ch[e] = sv + (corr ? bf2f(corr[e]) : 0.0f); }
    }
    __syncthreads();
    for (int k = 0; k < top; k++) {
        if (wave == 0) {
            float best = -INFINITY; int bi = 0x7FFFFFFF;
            for (int e = lane; e < n_all; e += 64) { const float v = ch[e]; if (v > best || (v == best && e < bi)) { best = v; bi = e; } }
            for (int o = 32; o > 0; o >>= 1) {
                const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(bi, o, 64);
                if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
            }
            if (lane == 0) { idx[(size_t)t * top + k] = bi; wgt[(size_t)t * top + k] = sc[bi]; ch[bi] = -INFINITY; }
        }
        __syncthreads();
    }
}

// grid (ff chunks, pairs): act[p][n] = gelu(W_up[e][n] . h[t]); a wave per n at a time.  Identity pairs do nothing.
template <bool GATED>
__global__ void __launch_bounds__(256) k_moe_up_rows(const float *__restrict__ h, size_t ldh, int W, int F, int experts, int top, const bf16_t *__restrict__ up,
                                                     const int *__restrict__ idx, float *__restrict__ act, int vec, int glu_kind, float limit)
{
    const int p = blockIdx.y, e = idx[p];
    if (e >= experts) return;
    const int lane = threadIdx.x & 63, wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), nwaves = gridDim.x * (blockDim.x >> 6);
    const float *hr = h + (size_t)(p / top) * ldh;
    if (GATED) {      // the expert's matrix holds F gate rows, then F up rows: both dots of an output side by side
        for (int n = wave; n < F; n += nwaves) {
            const bf16_t *wg = up + ((size_t)e * 2 * F + n) * W, *wu = wg + (size_t)F * W;
            float ag = 0.0f, au = 0.0f;
            if (vec) {
#pragma unroll 2
                for (int k = lane * 8; k < W; k += 512) {
                    const u32x4m gv = *reinterpret_cast<const u32x4m *>(wg + k), uv = *reinterpret_cast<const u32x4m *>(wu + k);
                    const float4 a0 = *reinterpret_cast<const float4 *>(hr + k), a1 = *reinterpret_cast<const float4 *>(hr + k + 4);
                    const float a8[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        ag = fmaf(a8[2 * j], __uint_as_float(gv[j] << 16), ag); ag = fmaf(a8[2 * j + 1], __uint_as_float(gv[j] & 0xFFFF0000u), ag);
                        au = fmaf(a8[2 * j], __uint_as_float(uv[j] << 16), au); au = fmaf(a8[2 * j + 1], __uint_as_float(uv[j] & 0xFFFF0000u), au);
                    }
                }
            } else {
                for (int k = lane; k < W; k += 64) { ag = fmaf(hr[k], bf2f(wg[k]), ag); au = fmaf(hr[k], bf2f(wu[k]), au); }
            }
            ag = wave_sum(ag); au = wave_sum(au);
            if (lane == 0) {
                if (glu_kind == 3) { const float g = fminf(ag, limit), u = fminf(fmaxf(au, -limit), limit); act[(size_t)p * F + n] = g * sigmoid_f(1.702f * g) * (u + 1.0f); }
                else act[(size_t)p * F + n] = silu_exact(ag) * au;
            }
        }
        return;
    }
    for (int n = wave; n < F; n += nwaves) {
        const bf16_t *w = up + ((size_t)e * F + n) * W;
        float acc = 0.0f;
        if (vec) {
#pragma unroll 4
            for (int k = lane * 8; k < W; k += 512) {
                const u32x4m wv = *reinterpret_cast<const u32x4m *>(w + k);
                const float4 a0 = *reinterpret_cast<const float4 *>(hr + k), a1 = *reinterpret_cast<const float4 *>(hr + k + 4);
                acc = fmaf(a0.x, __uint_as_float(wv[0] << 16), acc); acc = fmaf(a0.y, __uint_as_float(wv[0] & 0xFFFF0000u), acc);
                acc = fmaf(a0.z, __uint_as_float(wv[1] << 16), acc); acc = fmaf(a0.w, __uint_as_float(wv[1] & 0xFFFF0000u), acc);
                acc = fmaf(a1.x, __uint_as_float(wv[2] << 16), acc); acc = fmaf(a1.y, __uint_as_float(wv[2] & 0xFFFF0000u), acc);
                acc = fmaf(a1.z, __uint_as_float(wv[3] << 16), acc); acc = fmaf(a1.w, __uint_as_float(wv[3] & 0xFFFF0000u), acc);
            }
        } else {
            for (int k = lane; k < W; k += 64) acc = fmaf(hr[k], bf2f(w[k]), acc);
        }
        acc = wave_sum(acc);
        if (lane == 0) act[(size_t)p * F + n] = gelu_erf_f(acc);
    }
}

// grid (width chunks, rows): y[t][c] (+)= sum_k wgt * (identity ? h[t][c] : W_down[e][c] . act[p]); a wave per c at a time.  The chosen
// experts are walked eight at a time with their loads issued side by side (a step of one token is bound by requests in flight).
__global__ void __launch_bounds__(256) k_moe_down_rows(const float *__restrict__ h, size_t ldh, int W, int F, int experts, int top, const bf16_t *__restrict__ down,
                                                       const int *__restrict__ idx, const float *__restrict__ wgt, const float *__restrict__ act,
                                                       int accumulate, float *__restrict__ y, size_t ldy, int vec)
{
    const int t = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6), nwaves = gridDim.x * (blockDim.x >> 6);
    for (int c = wave; c < W; c += nwaves) {
        float out = 0.0f;
        for (int k0 = 0; k0 < top; k0 += 8) {
            int e[8]; float acc[8];
#pragma unroll
            for (int k = 0; k < 8; k++) { e[k] = k0 + k < top ? idx[t * top + k0 + k] : experts; acc[k] = 0.0f; }
            if (vec) {
                for (int j = lane * 8; j < F; j += 512) {
                    u32x4m wv[8]; float4 a0[8], a1[8];
#pragma unroll
                    for (int k = 0; k < 8; k++)
                        if (e[k] < experts) {
                            wv[k] = *reinterpret_cast<const u32x4m *>(down + ((size_t)e[k] * W + c) * F + j);
                            const float *a = act + (size_t)(t * top + k0 + k) * F + j;
                            a0[k] = *reinterpret_cast<const float4 *>(a); a1[k] = *reinterpret_cast<const float4 *>(a + 4);
                        }
#pragma unroll
                    for (int k = 0; k < 8; k++)
                        if (e[k] < experts) {
                            float s = acc[k];
                            s = fmaf(a0[k].x, __uint_as_float(wv[k][0] << 16), s); s = fmaf(a0[k].y, __uint_as_float(wv[k][0] & 0xFFFF0000u), s);
                            s = fmaf(a0[k].z, __uint_as_float(wv[k][1] << 16), s); s = fmaf(a0[k].w, __uint_as_float(wv[k][1] & 0xFFFF0000u), s);
                            s = fmaf(a1[k].x, __uint_as_float(wv[k][2] << 16), s); s = fmaf(a1[k].y, __uint_as_float(wv[k][2] & 0xFFFF0000u), s);
                            s = fmaf(a1[k].z, __uint_as_float(wv[k][3] << 16), s); s = fmaf(a1[k].w, __uint_as_float(wv[k][3] & 0xFFFF0000u), s);
                            acc[k] = s;
                        }
                }
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++)
                    if (e[k] < experts) {
                        const bf16_t *w = down + ((size_t)e[k] * W + c) * F;
                        const float *a = act + (size_t)(t * top + k0 + k) * F;
                        for (int j = lane; j < F; j += 64) acc[k] = fmaf(a[j], bf2f(w[j]), acc[k]);
                    }
            }
#pragma unroll
            for (int k = 0; k < 8; k++) {      // in the order of the row's choices
                if (k0 + k >= top) break;
                const float wk = wgt[t * top + k0 + k];
                out = fmaf(wk, e[k] < experts ? wave_sum(acc[k]) : h[(size_t)t * ldh + c], out);
            }
        }
        if (lane == 0) { float *d = y + (size_t)t * ldy + c; *d = accumulate ? *d + out : out; }
    }
}

// ONE workgroup: pairs (row, choice) sorted by expert.  a_rows[pos] = row of the pair at sorted place pos, pair_pos[p] = place of pair p
// (-1: identity), w_sorted[pos] = its weight, tile_map = tiles of at most 64 places of one expert, *n_tiles.  The place of a pair inside
// its expert's range comes from an LDS counter: the order there may differ from run to run, the values computed per pair do not.
__global__ void __launch_bounds__(1024) k_moe_sort(const int *__restrict__ idx, const float *__restrict__ wgt, int n_pairs, int experts, int top,
                                                   int *__restrict__ a_rows, int *__restrict__ pair_pos, float *__restrict__ w_sorted,
                                                   int *__restrict__ tile_map, int *__restrict__ n_tiles)
{
    extern __shared__ int cnt[];           // [experts] counts, then cursors; [experts + 1] offsets
    int *off = cnt + experts;
    for (int e = threadIdx.x; e < experts; e += blockDim.x) cnt[e] = 0;
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) { const int e = idx[p]; if (e < experts) atomicAdd(&cnt[e], 1); }
    __syncthreads();
    if (threadIdx.x == 0) {
        int o = 0, nt = 0;
        for (int e = 0; e < experts; e++) {
            off[e] = o;
            for (int r = 0; r < cnt[e]; r += 64) { tile_map[3 * nt] = e; tile_map[3 * nt + 1] = o + r; tile_map[3 * nt + 2] = min(64, cnt[e] - r); nt++; }
            o += cnt[e];
            cnt[e] = 0;
        }
        off[experts] = o;
        *n_tiles = nt;
    }
    __syncthreads();
    for (int p = threadIdx.x; p < n_pairs; p += blockDim.x) {
        const int e = idx[p];
        if (e >= experts) { pair_pos[p] = -1; continue; }
        const int pos = off[e] + atomicAdd(&cnt[e], 1);
        a_rows[pos] = p / top; pair_pos[p] = pos; w_sorted[pos] = wgt[p];
    }
}

// y[t][c] (+)= sum_k (identity ? wgt h[t][c] : yp[pair_pos][c])  (the pair's weight is already inside yp)
__global__ void __launch_bounds__(256) k_moe_combine(const float *__restrict__ h, size_t ldh, int W, int top, const int *__restrict__ pair_pos,
                                                     const float *__restrict__ wgt, const float *__restrict__ yp, int accumulate, float *__restrict__ y, size_t ldy)
{
    const int t = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= W) return;
    float out = 0.0f;
    for (int k = 0; k < top; k++) {
        const int p = t * top + k, pos = pair_pos[p];
        out += pos < 0 ? wgt[p] * h[(size_t)t * ldh + c] : yp[(size_t)pos * W + c];
    }
    float *d = y + (size_t)t * ldy + c;
    *d = accumulate ? *d + out : out;
}

size_t al16(size_t v) { return (v + 15) & ~(size_t)15; }
size_t moe_tiles_max(size_t rows, int top, int experts) { return (rows * (size_t)top + 63) / 64 + (size_t)experts; }

} // namespace

extern "C" {

int ifa_moe_route_scores_f32(int score_kind, const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *correction_bf16, int *idx_dev,
                             void *wgt_f32, ifa_stream stream)
{
    IFA_REQUIRE(logits_f32 && idx_dev && wgt_f32, "ifa_moe_route_scores_f32: null pointer");
    IFA_REQUIRE(rows > 0 && n_all >= 1 && n_all <= 4096 && top >= 1 && top <= n_all && ld >= (size_t)n_all && (score_kind == 0 || score_kind == 1),
                "ifa_moe_route_scores_f32: bad shape (%d router outputs, %d chosen, scores of kind %d)", n_all, top, score_kind);
    hipLaunchKernelGGL(k_moe_route, dim3((unsigned)rows), dim3(64), (size_t)n_all * 8, ifa_s(stream), (const float *)logits_f32, ld, n_all, top,
                       (const bf16_t *)correction_bf16, idx_dev, (float *)wgt_f32, score_kind);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_moe_route_f32(const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *correction_bf16, int *idx_dev, void *wgt_f32,
                      ifa_stream stream)
{
    return ifa_moe_route_scores_f32(0, logits_f32, ld, rows, n_all, top, correction_bf16, idx_dev, wgt_f32, stream);
}

int ifa_moe_route_rows_f32(const void *h_f32, size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top, const void *correction_bf16,
                           int *idx_dev, void *wgt_f32, ifa_stream stream)
{
    return ifa_moe_route_rows_scores_f32(0, h_f32, ldh, rows, width, router_bf16, n_all, top, correction_bf16, idx_dev, wgt_f32, stream);
}

int ifa_moe_route_rows_scores_f32(int score_kind, const void *h_f32, size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top,
                                  const void *correction_bf16, int *idx_dev, void *wgt_f32, ifa_stream stream)
{
    IFA_REQUIRE(h_f32 && router_bf16 && idx_dev && wgt_f32, "ifa_moe_route_rows_f32: null pointer");
    IFA_REQUIRE(rows > 0 && rows <= 64 && width > 0 && n_all >= 1 && n_all <= 4096 && top >= 1 && top <= n_all && ldh >= (size_t)width && (score_kind == 0 || score_kind == 1),
                "ifa_moe_route_rows_f32: bad shape");
    const int vec = (width % 8 == 0 && ldh % 4 == 0 && ((uintptr_t)h_f32 & 15) == 0 && ((uintptr_t)router_bf16 & 15) == 0) ? 1 : 0;
    hipLaunchKernelGGL(k_moe_route_rows, dim3((unsigned)rows), dim3(n_all > 8 ? 1024 : 256), (size_t)n_all * 8, ifa_s(stream), (const float *)h_f32, ldh, width,
                       (const bf16_t *)router_bf16, n_all, top, (const bf16_t *)correction_bf16, idx_dev, (float *)wgt_f32, vec, score_kind, (const float *)nullptr, (size_t)0,
                       (const bf16_t *)nullptr, (const bf16_t *)nullptr, (const bf16_t *)nullptr, (float *)nullptr);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_moe_dyt_route_rows_f32(int score_kind, const void *x_f32, size_t ldx, const void *alpha_bf16, const void *norm_w_bf16, const void *norm_b_bf16, void *h_f32,
                               size_t ldh, size_t rows, int width, const void *router_bf16, int n_all, int top, const void *correction_bf16, int *idx_dev,
                               void *wgt_f32, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && alpha_bf16 && norm_w_bf16 && norm_b_bf16 && h_f32 && router_bf16 && idx_dev && wgt_f32 && x_f32 != h_f32, "ifa_moe_dyt_route_rows_f32: null pointer");
    IFA_REQUIRE(rows > 0 && rows <= 64 && width > 0 && n_all >= 1 && n_all <= 4096 && top >= 1 && top <= n_all && ldh >= (size_t)width && ldx >= (size_t)width
                && (score_kind == 0 || score_kind == 1), "ifa_moe_dyt_route_rows_f32: bad shape");
    const int vec = (width % 8 == 0 && ldh % 4 == 0 && ((uintptr_t)h_f32 & 15) == 0 && ((uintptr_t)router_bf16 & 15) == 0) ? 1 : 0;
    hipLaunchKernelGGL(k_moe_route_rows, dim3((unsigned)rows), dim3(n_all > 8 ? 1024 : 256), (size_t)n_all * 8, ifa_s(stream), (const float *)h_f32, ldh, width,
                       (const bf16_t *)router_bf16, n_all, top, (const bf16_t *)correction_bf16, idx_dev, (float *)wgt_f32, vec, score_kind, (const float *)x_f32, ldx,
                       (const bf16_t *)alpha_bf16, (const bf16_t *)norm_w_bf16, (const bf16_t *)norm_b_bf16, (float *)h_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_moe_route_top_f32(const void *logits_f32, size_t ld, size_t rows, int n_all, int top, const void *bias_bf16, int *idx_dev, void *wgt_f32,
                          ifa_stream stream)
{
    IFA_REQUIRE(logits_f32 && idx_dev && wgt_f32, "ifa_moe_route_top_f32: null pointer");
    IFA_REQUIRE(rows > 0 && n_all >= 1 && n_all <= 4096 && top >= 1 && top <= n_all && ld >= (size_t)n_all, "ifa_moe_route_top_f32: bad shape (%d router outputs, %d chosen)", n_all, top);
    hipLaunchKernelGGL(k_moe_route_top, dim3((unsigned)rows), dim3(64), (size_t)(n_all + top) * 4, ifa_s(stream), (const float *)logits_f32, ld, n_all, top,
                       (const bf16_t *)bias_bf16, idx_dev, (float *)wgt_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

size_t ifa_moe_workspace_bytes(size_t rows, int top, int width, int ff, int experts)
{
    const size_t pairs = rows * (size_t)top;
    return al16(pairs * ff * 4) + al16(pairs * width * 4) + 3 * al16(pairs * 4) + al16(moe_tiles_max(rows, top, experts) * 12) + 16;
}

static int moe_experts(const char *who, int gated, int glu_kind, float limit, const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int identity, int top, int act,
                       const void *up_bf16, const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes,
                       void *y_f32, size_t ldy, int accumulate, ifa_stream stream)
{
    IFA_REQUIRE(h_f32 && idx_dev && wgt_f32 && ws && y_f32 && (experts == 0 || (up_bf16 && down_bf16)), "%s: null pointer", who);
    IFA_REQUIRE(rows > 0 && rows < 65536 && width > 0 && ff > 0 && experts >= 0 && experts <= 4096 && identity >= 0 && top >= 1 && top <= experts + identity && act == 0
                && ldh >= (size_t)width && ldy >= (size_t)width, "%s: bad shape", who);
    // gated experts: the first product leaves gate | up (2 ff values per pair) in front of the activations
    const int ff_ws = gated ? 3 * ff : ff;
    IFA_REQUIRE(ws_bytes >= ifa_moe_workspace_bytes(rows, top, width, ff_ws, experts) && ((uintptr_t)ws & 15) == 0, "%s: workspace of %zu bytes, %zu needed", who, ws_bytes,
                ifa_moe_workspace_bytes(rows, top, width, ff_ws, experts));
    const size_t pairs = rows * (size_t)top;
    char *b = (char *)ws;
    float *actb = (float *)b; b += al16(pairs * ff_ws * 4);
    float *gub = actb + pairs * ff;                     // [pairs][2 ff] (gated experts, many rows)
    float *yp = (float *)b; b += al16(pairs * width * 4);
    int *a_rows = (int *)b; b += al16(pairs * 4);
    int *pair_pos = (int *)b; b += al16(pairs * 4);
    float *w_sorted = (float *)b; b += al16(pairs * 4);
    int *tile_map = (int *)b; b += al16(moe_tiles_max(rows, top, experts) * 12);
    int *n_tiles = (int *)b;
    hipStream_t s = ifa_s(stream);
    const float *h = (const float *)h_f32;
    if (rows <= 8 || experts == 0) {
        const int vec_u = (width % 8 == 0 && ldh % 4 == 0 && ((uintptr_t)h_f32 & 15) == 0 && ((uintptr_t)up_bf16 & 15) == 0) ? 1 : 0;
        const int vec_d = (ff % 8 == 0 && ((uintptr_t)down_bf16 & 15) == 0) ? 1 : 0;
        if (experts > 0 && gated)
            hipLaunchKernelGGL(k_moe_up_rows<true>, dim3(std::min(512u, ifa_cdiv((size_t)ff, 4)), (unsigned)pairs), dim3(256), 0, s, h, ldh, width, ff, experts, top,
                               (const bf16_t *)up_bf16, idx_dev, actb, vec_u, glu_kind, limit);
        else if (experts > 0)
            hipLaunchKernelGGL(k_moe_up_rows<false>, dim3(std::min(512u, ifa_cdiv((size_t)ff, 4)), (unsigned)pairs), dim3(256), 0, s, h, ldh, width, ff, experts, top,
                               (const bf16_t *)up_bf16, idx_dev, actb, vec_u, 0, 0.0f);
        hipLaunchKernelGGL(k_moe_down_rows, dim3(std::min(1024u, ifa_cdiv((size_t)width, 4)), (unsigned)rows), dim3(256), 0, s, h, ldh, width, ff, experts, top,
                           (const bf16_t *)down_bf16, idx_dev, (const float *)wgt_f32, actb, accumulate ? 1 : 0, (float *)y_f32, ldy, vec_d);
        IFA_LAUNCH_CHECK();
        return IFA_OK;
    }
    const size_t max_tiles = moe_tiles_max(rows, top, experts);
    IFA_REQUIRE(max_tiles < 65536, "%s: %zu rows x %d choices exceed one step", who, rows, top);
    hipLaunchKernelGGL(k_moe_sort, dim3(1), dim3(1024), (size_t)(2 * experts + 1) * 4, s, idx_dev, (const float *)wgt_f32, (int)pairs, experts, top, a_rows, pair_pos, w_sorted,
                       tile_map, n_tiles);
    IFA_LAUNCH_CHECK();
    int rc;
    if (gated) {
        if ((rc = ifa_linear_bf16w_grouped(up_bf16, (size_t)2 * ff, (size_t)width, experts, h_f32, ldh, a_rows, tile_map, n_tiles, max_tiles, nullptr, 0, ops32, gub, (size_t)2 * ff, stream))) return rc;
        if ((rc = ifa_glu_ex_f32(glu_kind, limit, gub, (size_t)2 * ff, pairs, (size_t)ff, nullptr, 0, actb, (size_t)ff, stream))) return rc;
    } else
    if ((rc = ifa_linear_bf16w_grouped(up_bf16, (size_t)ff, (size_t)width, experts, h_f32, ldh, a_rows, tile_map, n_tiles, max_tiles, nullptr, 1, ops32, actb, (size_t)ff, stream))) return rc;
    if ((rc = ifa_linear_bf16w_grouped(down_bf16, (size_t)width, (size_t)ff, experts, actb, (size_t)ff, nullptr, tile_map, n_tiles, max_tiles, w_sorted, 0, ops32, yp, (size_t)width, stream))) return rc;
    hipLaunchKernelGGL(k_moe_combine, dim3(ifa_cdiv((size_t)width, 256), (unsigned)rows), dim3(256), 0, s, h, ldh, width, top, pair_pos, (const float *)wgt_f32, yp,
                       accumulate ? 1 : 0, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_moe_experts_f32(const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int identity, int top, int act,
                        const void *up_bf16, const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes,
                        void *y_f32, size_t ldy, int accumulate, ifa_stream stream)
{
    return moe_experts("ifa_moe_experts_f32", 0, 0, 0.0f, h_f32, ldh, rows, width, ff, experts, identity, top, act, up_bf16, down_bf16, idx_dev, wgt_f32, ops32, ws, ws_bytes, y_f32,
                       ldy, accumulate, stream);
}

int ifa_moe_experts_gated_f32(const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int top, const void *gate_up_bf16,
                              const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes, void *y_f32, size_t ldy,
                              int accumulate, ifa_stream stream)
{
    IFA_REQUIRE(experts > 0, "ifa_moe_experts_gated_f32: no experts");
    return moe_experts("ifa_moe_experts_gated_f32", 1, 0, 0.0f, h_f32, ldh, rows, width, ff, experts, 0, top, 0, gate_up_bf16, down_bf16, idx_dev, wgt_f32, ops32, ws, ws_bytes,
                       y_f32, ldy, accumulate, stream);
}

int ifa_moe_experts_glu_f32(int glu_kind, float limit, const void *h_f32, size_t ldh, size_t rows, int width, int ff, int experts, int top,
                            const void *gate_up_bf16, const void *down_bf16, const int *idx_dev, const void *wgt_f32, int ops32, void *ws, size_t ws_bytes,
                            void *y_f32, size_t ldy, int accumulate, ifa_stream stream)
{
    IFA_REQUIRE(experts > 0 && (glu_kind == 0 || (glu_kind == 3 && limit > 0.0f)), "ifa_moe_experts_glu_f32: no experts, or gate kind %d (0, or 3 with a limit)", glu_kind);
    return moe_experts("ifa_moe_experts_glu_f32", 1, glu_kind, limit, h_f32, ldh, rows, width, ff, experts, 0, top, 0, gate_up_bf16, down_bf16, idx_dev, wgt_f32, ops32, ws,
                       ws_bytes, y_f32, ldy, accumulate, stream);
}

} // extern "C"
