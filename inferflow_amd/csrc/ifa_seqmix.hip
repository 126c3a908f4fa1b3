// ifa_seqmix.hip -- sequence mixers with a recurrent state instead of a key / value cache, on 32-bit activations:
//   * short causal convolution per channel + SiLU (+ unit-norm of head groups), its tail carried per sequence
//   * per-head matrix state S [dk][dv] advanced token by token:
//       kind 0  linear attention with a constant decay per head:  S <- d S + k v^T;                      o = S^T q
//     (in_act = 1: q, k, v pass SiLU as they are read)
//       kind 1  gated delta rule:                                 S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//   * the gates of the delta rule (beta = sigmoid, g = exp(-exp(A_log) softplus(a + dt_bias)))
//   * the generalized delta rule with a decay w and a removal rate per key channel: S <- diag(w) S - b (u^T S) + k v^T, o = S^T q
//     (u the unit key, b = removal rate * u), and its gates
//   * RMS norm over channel groups with a weight and an output gate (sigmoid or SiLU)
// Everything that enters a recurrence is fp32; states live in fp32 in the slot arena of the worker (a table of one
// base pointer per slot + an offset per layer).  A sequence that starts at position 0 starts from a zero state,
// whatever the slot held before.
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"

using namespace ifa32;

namespace {

// grid: (rows, channel slices).  y[t][c] = silu(sum_j w[c][j] in(i - (taps - 1) + j)[c]); in(idx) for idx < 0 comes from the
// sequence's carried tail (rows [taps - 1][C], oldest first) or is zero at the start of a sequence.  Then channels
// [0, norm_cols) are turned into unit vectors in groups of gdim (x / sqrt(sum x^2 + l2_eps)) and channels [0, scale_cols)
// are multiplied by qscale.
__global__ void __launch_bounds__(256) k_shortconv_silu(const float *__restrict__ x, size_t ldx, int C, int taps, const bf16_t *__restrict__ w,
                                                        const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq,
                                                        float *const *__restrict__ slot_base, size_t state_off, int norm_cols, int gdim,
                                                        float l2_eps, int scale_cols, float qscale, float *__restrict__ y, size_t ldy, int slice)
{
    extern __shared__ float ys[];
    const int t = blockIdx.x;
    const int c_lo = blockIdx.y * slice, c_hi = min(C, c_lo + slice);      // this workgroup's channels (whole norm groups: slice % gdim == 0)
    const SeqDesc sd = seqs[row_seq[t]];
    const int i = t - sd.row0;
    const float *tail = sd.pos0 > 0 ? slot_base[sd.slot] + state_off : nullptr;
    for (int c = c_lo + threadIdx.x; c < c_hi; c += blockDim.x) {
        float acc = 0.0f;
        for (int j = 0; j < taps; j++) {
            const int idx = i - (taps - 1) + j;
            float v;
            if (idx >= 0) v = x[(size_t)(sd.row0 + idx) * ldx + c];
            else v = tail ? tail[(size_t)(taps - 1 + idx) * C + c] : 0.0f;
            acc = fmaf(bf2f(w[(size_t)c * taps + j]), v, acc);
        }
        ys[c - c_lo] = silu_exact(acc);
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int g_lo = gdim > 0 ? c_lo / gdim : 0, g_hi = gdim > 0 ? min(norm_cols, c_hi) / gdim : 0;
    for (int gidx = g_lo + wave; gidx < g_hi; gidx += nw) {
        float s = 0.0f;
        for (int e = lane; e < gdim; e += 64) { const float v = ys[gidx * gdim + e - c_lo]; s = fmaf(v, v, s); }
        s = wave_sum(s);
        const float r = 1.0f / sqrtf(s + l2_eps);
        for (int e = lane; e < gdim; e += 64) ys[gidx * gdim + e - c_lo] *= r;
    }
    __syncthreads();
    for (int c = c_lo + threadIdx.x; c < c_hi; c += blockDim.x) y[(size_t)t * ldy + c] = c < scale_cols ? ys[c - c_lo] * qscale : ys[c - c_lo];
}

// y[t][c] = x[t][c] + sum_j w[c][j] * x_(t - taps + 1 + j)[c]: the same causal taps without activation, added to the input itself
__global__ void __launch_bounds__(256) k_shortconv_residual(const float *__restrict__ x, size_t ldx, int C, int taps, const bf16_t *__restrict__ w,
                                                            const SeqDesc *__restrict__ seqs, const int *__restrict__ row_seq,
                                                            float *const *__restrict__ slot_base, size_t state_off, float *__restrict__ y, size_t ldy)
{
    const int t = blockIdx.x;
    const SeqDesc sd = seqs[row_seq[t]];
    const int i = t - sd.row0;
    const float *tail = sd.pos0 > 0 ? slot_base[sd.slot] + state_off : nullptr;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < C; c += gridDim.y * blockDim.x) {
        float acc = 0.0f;
        for (int j = 0; j < taps; j++) {
            const int idx = i - (taps - 1) + j;
            float v;
            if (idx >= 0) v = x[(size_t)(sd.row0 + idx) * ldx + c];
            else v = tail ? tail[(size_t)(taps - 1 + idx) * C + c] : 0.0f;
            acc = fmaf(bf2f(w[(size_t)c * taps + j]), v, acc);
        }
        y[(size_t)t * ldy + c] = x[(size_t)t * ldx + c] + acc;
    }
}

// Steps of a few rows: what lies between two sub-layers of a post-norm block in one launch --
//   1. x[t] += m[t] / sqrt(mean_part(m[t]^2) + eps) * nw          (grouped RMS norm of a sub-layer's output into the residual; m null: skip)
//   2. stack[count - 1] <- x; x <- sum_j dw[j] stack[j]            (depth average; stack null: skip)
//   3. h[t] = x[t] + conv(x)[t]                                    (input convolution of the next sub-layer; cw null: skip)
//   4. the convolution's carried tail advanced past the step's rows
// A workgroup per norm part: stages 2 to 4 work channel by channel, stage 1 within a part, so a part's channels [c_lo, c_hi) never
// meet another part's and the barriers between the stages are the workgroup's own.
__global__ void __launch_bounds__(256) k_norm_add_conv_rows(float *__restrict__ x, int T, int W, const float *__restrict__ m, size_t ldm, const bf16_t *__restrict__ nw,
                                                            int groups, float eps, float *__restrict__ stack, size_t plane, int count, const bf16_t *__restrict__ dw,
                                                            const bf16_t *__restrict__ cw, int taps, const SeqDesc *__restrict__ seqs, int nseq,
                                                            const int *__restrict__ row_seq, float *const *__restrict__ slot_base, size_t state_off,
                                                            float *__restrict__ h)
{
    __shared__ float red[17];
    const int tid = threadIdx.x, gs = W / groups, c_lo = blockIdx.x * gs, c_hi = c_lo + gs;
    if (m) {
        for (int t = 0; t < T; t++) {
            const float *mr = m + (size_t)t * ldm;
            float q = 0.0f;
            for (int c = c_lo + tid; c < c_hi; c += blockDim.x) q = fmaf(mr[c], mr[c], q);
            const float rinv = 1.0f / sqrtf(block_sum(q, red) / (float)gs + eps);
            for (int c = c_lo + tid; c < c_hi; c += blockDim.x) {
                float v = mr[c] * rinv;
                if (nw) v *= bf2f(nw[c]);
                x[(size_t)t * W + c] += v;
            }
        }
    }
    // (from here on a thread only meets values of its own channels: what it wrote above it reads back itself)
    if (stack) {
        for (int t = 0; t < T; t++)
            for (int c = c_lo + tid; c < c_hi; c += blockDim.x) {
                const size_t i = (size_t)t * W + c;
                const float cur = x[i];
                stack[(size_t)(count - 1) * plane + i] = cur;
                float s = 0.0f;
                for (int j = 0; j + 1 < count; j++) s = fmaf(bf2f(dw[j]), stack[(size_t)j * plane + i], s);
                x[i] = fmaf(bf2f(dw[count - 1]), cur, s);
            }
    }
    if (!cw) return;
    for (int t = 0; t < T; t++) {
        const SeqDesc sd = seqs[row_seq[t]];
        const int i = t - sd.row0;
        const float *tail = sd.pos0 > 0 ? slot_base[sd.slot] + state_off : nullptr;
        for (int c = c_lo + tid; c < c_hi; c += blockDim.x) {
            float acc = 0.0f;
            for (int j = 0; j < taps; j++) {
                const int idx = i - (taps - 1) + j;
                float v;
                if (idx >= 0) v = x[(size_t)(sd.row0 + idx) * W + c];
                else v = tail ? tail[(size_t)(taps - 1 + idx) * W + c] : 0.0f;
                acc = fmaf(bf2f(cw[(size_t)c * taps + j]), v, acc);
            }
            h[(size_t)t * W + c] = x[(size_t)t * W + c] + acc;
        }
    }
    const int keep = taps - 1;
    for (int q = 0; q < nseq; q++) {
        const SeqDesc sd = seqs[q];
        float *tail = slot_base[sd.slot] + state_off;
        for (int c = c_lo + tid; c < c_hi; c += blockDim.x)
            for (int r = 0; r < keep; r++) {          // ascending r: a value read from the old tail lies above what was written so far
                const int idx = sd.n - keep + r;
                float v;
                if (idx >= 0) v = x[(size_t)(sd.row0 + idx) * W + c];
                else v = sd.pos0 > 0 ? tail[(size_t)(keep + idx) * W + c] : 0.0f;
                tail[(size_t)r * W + c] = v;
            }
    }
}

// grid: one workgroup per sequence.  The carried tail becomes the last taps - 1 inputs of (old tail, this step's rows).
__global__ void __launch_bounds__(256) k_shortconv_tail(const float *__restrict__ x, size_t ldx, int C, int taps, const SeqDesc *__restrict__ seqs,
                                                        float *const *__restrict__ slot_base, size_t state_off)
{
    const SeqDesc sd = seqs[blockIdx.x];
    float *tail = slot_base[sd.slot] + state_off;
    const int keep = taps - 1;
    for (int c = threadIdx.x; c < C; c += blockDim.x)
        for (int r = 0; r < keep; r++) {          // ascending r: a value read from the old tail lies above what was written so far
            const int idx = sd.n - keep + r;      // index into this step's rows
            float v;
            if (idx >= 0) v = x[(size_t)(sd.row0 + idx) * ldx + c];
            else v = sd.pos0 > 0 ? tail[(size_t)(keep + idx) * C + c] : 0.0f;
            tail[(size_t)r * C + c] = v;
        }
}

// beta[t][h] = sigmoid(b[t][h]);  g[t][h] = exp(-exp(A_log[h]) * softplus(a[t][h] + dt_bias[h]))
__global__ void __launch_bounds__(256) k_delta_gates(const float *__restrict__ b, size_t ldb, const float *__restrict__ a, size_t lda, int H, int T,
                                                     const bf16_t *__restrict__ A_log, const bf16_t *__restrict__ dt_bias, float *__restrict__ beta,
                                                     float *__restrict__ g)
{
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= T * H) return;
    const int t = idx / H, h = idx % H;
    beta[idx] = sigmoid_f(b[(size_t)t * ldb + h]);
    g[idx] = expf(-expf(bf2f(A_log[h])) * softplus_f(a[(size_t)t * lda + h] + bf2f(dt_bias[h])));
}

struct ScanArgs {
    const float *q, *k, *v; size_t ldq, ldk, ldv;
    int heads, qk_heads, dk, dv, in_act;
    const float *decay_head, *decay_row, *beta_row;
    const SeqDesc *seqs; float *const *slot_base; size_t state_off;
    float *out; size_t ldo;
};

constexpr int SCAN_DKL = 4;       // dk <= 64 * SCAN_DKL

// grid (sequences * heads, ceil(dv / 64)), one wave per workgroup: the columns of S are independent in both recurrences, so
// each lane owns one column S[:, j] (in LDS, [dk][64]: conflict-free) and needs q_t, k_t (broadcast from LDS) and its v_t[j].
// The next token's operands are requested before the current token is computed.
template <int KIND>
__global__ void __launch_bounds__(64) k_state_scan(ScanArgs P)
{
    extern __shared__ float sm[];
    float *S = sm, *qs = sm + (size_t)P.dk * 64, *ks = qs + P.dk;
    const int seq = blockIdx.x / P.heads, h = blockIdx.x % P.heads;
    const int lane = threadIdx.x, j = blockIdx.y * 64 + lane;
    const bool live = j < P.dv;
    const int jc = live ? j : P.dv - 1;
    const int qh = h / (P.heads / P.qk_heads);
    const SeqDesc sd = P.seqs[seq];
    float *state = P.slot_base[sd.slot] + P.state_off + (size_t)h * P.dk * P.dv;
    const int dk = P.dk;
    if (sd.pos0 > 0) for (int i = 0; i < dk; i++) S[i * 64 + lane] = state[(size_t)i * P.dv + jc];
    else for (int i = 0; i < dk; i++) S[i * 64 + lane] = 0.0f;
    const float dconst = KIND == 0 ? P.decay_head[h] : 0.0f;
    float qr[SCAN_DKL], kr[SCAN_DKL], vr, gr = 0.0f, br = 0.0f;
    auto request = [&](int t) {
        const size_t row = (size_t)(sd.row0 + t);
#pragma unroll
        for (int e = 0; e < SCAN_DKL; e++) {
            const int i = lane + 64 * e;
            if (i < dk) {
                qr[e] = P.q[row * P.ldq + (size_t)qh * dk + i]; kr[e] = P.k[row * P.ldk + (size_t)qh * dk + i];
                if (P.in_act) { qr[e] = silu_exact(qr[e]); kr[e] = silu_exact(kr[e]); }
            }
        }
        vr = P.v[row * P.ldv + (size_t)h * P.dv + jc];
        if (P.in_act) vr = silu_exact(vr);
        if (KIND == 1) { gr = P.decay_row[row * P.heads + h]; br = P.beta_row[row * P.heads + h]; }
    };
    if (sd.n > 0) request(0);
    for (int t = 0; t < sd.n; t++) {
        __syncthreads();          // the previous token's reads of qs / ks are done
#pragma unroll
        for (int e = 0; e < SCAN_DKL; e++) { const int i = lane + 64 * e; if (i < dk) { qs[i] = qr[e]; ks[i] = kr[e]; } }
        const float vt = vr, gt = gr, bt = br;
        __syncthreads();
        if (t + 1 < sd.n) request(t + 1);
        float o = 0.0f;
        if (KIND == 0) {
            for (int i = 0; i < dk; i++) {
                const float s = fmaf(dconst, S[i * 64 + lane], ks[i] * vt);
                S[i * 64 + lane] = s;
                o = fmaf(s, qs[i], o);
            }
        } else {
            float r = 0.0f;
            for (int i = 0; i < dk; i++) {
                const float s = gt * S[i * 64 + lane];
                S[i * 64 + lane] = s;
                r = fmaf(s, ks[i], r);
            }
            const float u = bt * (vt - r);
            for (int i = 0; i < dk; i++) {
                const float s = fmaf(ks[i], u, S[i * 64 + lane]);
                S[i * 64 + lane] = s;
                o = fmaf(s, qs[i], o);
            }
        }
        if (live) P.out[(size_t)(sd.row0 + t) * P.ldo + (size_t)h * P.dv + j] = o;
    }
    if (live) for (int i = 0; i < dk; i++) state[(size_t)i * P.dv + j] = S[i * 64 + lane];
}

// The same recurrences for key sizes 16 / 32 / 64 / 128 with the state in REGISTERS and FOUR (key sizes from 64 on: EIGHT) lanes per column:
// lane 4 c + r of a wave owns rows [r DK / 4, (r + 1) DK / 4) of column c (16 columns per wave), so a token is DK / 4 elements of dependent arithmetic per lane
// instead of DK -- the recurrence is a chain of dependent instructions of a wave that is alone on its SIMD, and its length per token
// is what the prompt rate of these layers comes down to.  The sums over a column's rows (the read-out, and S^T k of the delta rule)
// are finished across the lanes of a column by two DPP quad permutes (+ one half-row mirror for eight lanes).  Tokens go in groups of 8: the group's q, k and gates are staged in
// LDS (16-byte reads of a lane's row range), the next group's operands are requested from memory before the current group is
// computed.  fp32 results differ from the general kernel's by the order of these sums only.
constexpr int SCAN_TB = 8;

template <int KIND, int DK, int LPC>
__global__ void __launch_bounds__(64) k_state_scan_reg(ScanArgs P)
{
    constexpr int DKQ = DK / LPC, CPW = 64 / LPC;      // rows per lane, columns per wave
    __shared__ __attribute__((aligned(16))) float qs[2][SCAN_TB][DK], ks[2][SCAN_TB][DK];
    __shared__ float gs[2][SCAN_TB], bs[2][SCAN_TB];
    const int seq = blockIdx.x / P.heads, h = blockIdx.x % P.heads;
    const int lane = threadIdx.x, rg = lane & (LPC - 1), j = blockIdx.y * CPW + lane / LPC;
    const bool live = j < P.dv;
    const int jc = live ? j : P.dv - 1;
    const int qh = h / (P.heads / P.qk_heads);
    const SeqDesc sd = P.seqs[seq];
    float *state = P.slot_base[sd.slot] + P.state_off + ((size_t)h * DK + (size_t)rg * DKQ) * P.dv;
    float S[DKQ];
    if (sd.pos0 > 0) {
#pragma unroll
        for (int e = 0; e < DKQ; e++) S[e] = state[(size_t)e * P.dv + jc];
    } else {
#pragma unroll
        for (int e = 0; e < DKQ; e++) S[e] = 0.0f;
    }
    const float dconst = KIND == 0 ? P.decay_head[h] : 0.0f;
    constexpr int PER = SCAN_TB * DK / 64;          // q (and k) values of a group per lane
    float qr[PER], kr[PER], vnext[SCAN_TB], vcur[SCAN_TB], gr = 0.0f, br = 0.0f;
    auto request = [&](int t0) {                    // the group that starts at token t0 -> registers
#pragma unroll
        for (int u = 0; u < PER; u++) {
            const int e = lane + 64 * u, tt = e / DK, i = e % DK;
            const size_t row = (size_t)(sd.row0 + min(t0 + tt, sd.n - 1));
            qr[u] = P.q[row * P.ldq + (size_t)qh * DK + i]; kr[u] = P.k[row * P.ldk + (size_t)qh * DK + i];
            if (P.in_act) { qr[u] = silu_exact(qr[u]); kr[u] = silu_exact(kr[u]); }
        }
#pragma unroll
        for (int tt = 0; tt < SCAN_TB; tt++) {
            const size_t row = (size_t)(sd.row0 + min(t0 + tt, sd.n - 1));
            vnext[tt] = P.v[row * P.ldv + (size_t)h * P.dv + jc];
            if (P.in_act) vnext[tt] = silu_exact(vnext[tt]);
        }
        if (KIND == 1 && lane < SCAN_TB) {
            const size_t row = (size_t)(sd.row0 + min(t0 + lane, sd.n - 1));
            gr = P.decay_row[row * P.heads + h]; br = P.beta_row[row * P.heads + h];
        }
    };
    auto publish = [&](int buf) {                   // registers -> LDS buffer
#pragma unroll
        for (int u = 0; u < PER; u++) { const int e = lane + 64 * u; qs[buf][e / DK][e % DK] = qr[u]; ks[buf][e / DK][e % DK] = kr[u]; }
        if (KIND == 1 && lane < SCAN_TB) { gs[buf][lane] = gr; bs[buf][lane] = br; }
#pragma unroll
        for (int tt = 0; tt < SCAN_TB; tt++) vcur[tt] = vnext[tt];
    };
    if (sd.n > 0) { request(0); publish(0); }
    __syncthreads();
    for (int t0 = 0, buf = 0; t0 < sd.n; t0 += SCAN_TB, buf ^= 1) {
        const bool more = t0 + SCAN_TB < sd.n;
        if (more) request(t0 + SCAN_TB);
        const int cnt = min(SCAN_TB, sd.n - t0);
#pragma unroll
        for (int tt = 0; tt < SCAN_TB; tt++) {
            if (tt < cnt) {
                const float vt = vcur[tt];
                float kk[DKQ], qq[DKQ];
#pragma unroll
                for (int e4 = 0; e4 < DKQ; e4 += 4) {
                    const float4 k4 = *reinterpret_cast<const float4 *>(&ks[buf][tt][rg * DKQ + e4]), q4 = *reinterpret_cast<const float4 *>(&qs[buf][tt][rg * DKQ + e4]);
                    kk[e4] = k4.x; kk[e4 + 1] = k4.y; kk[e4 + 2] = k4.z; kk[e4 + 3] = k4.w;
                    qq[e4] = q4.x; qq[e4 + 1] = q4.y; qq[e4 + 2] = q4.z; qq[e4 + 3] = q4.w;
                }
                float o0 = 0.0f, o1 = 0.0f;
                if (KIND == 0) {
#pragma unroll
                    for (int e = 0; e < DKQ; e += 2) {
                        S[e] = fmaf(dconst, S[e], kk[e] * vt); o0 = fmaf(S[e], qq[e], o0);
                        S[e + 1] = fmaf(dconst, S[e + 1], kk[e + 1] * vt); o1 = fmaf(S[e + 1], qq[e + 1], o1);
                    }
                } else {
                    const float gt = gs[buf][tt], bt = bs[buf][tt];
                    float r0 = 0.0f, r1 = 0.0f;
#pragma unroll
                    for (int e = 0; e < DKQ; e += 2) {
                        S[e] *= gt; r0 = fmaf(S[e], kk[e], r0);
                        S[e + 1] *= gt; r1 = fmaf(S[e + 1], kk[e + 1], r1);
                    }
                    const float u = bt * (vt - (LPC == 8 ? oct_sum(r0 + r1) : quad_sum(r0 + r1)));
#pragma unroll
                    for (int e = 0; e < DKQ; e += 2) {
                        S[e] = fmaf(kk[e], u, S[e]); o0 = fmaf(S[e], qq[e], o0);
                        S[e + 1] = fmaf(kk[e + 1], u, S[e + 1]); o1 = fmaf(S[e + 1], qq[e + 1], o1);
                    }
                }
                const float o = LPC == 8 ? oct_sum(o0 + o1) : quad_sum(o0 + o1);
                if (live && rg == 0) P.out[(size_t)(sd.row0 + t0 + tt) * P.ldo + (size_t)h * P.dv + j] = o;
            }
        }
        if (more) publish(buf ^ 1);     // (the other buffer was last read one group ago, before the barrier below)
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int e = 0; e < DKQ; e++) state[(size_t)e * P.dv + j] = S[e];
    }
}

// ---- generalized delta rule with a decay and a removal rate per key channel:
//   S <- diag(w_t) S - b_t (u_t^T S) + k_t v_t^T   (both terms read the old state),   o_t = S^T q_t
// w (decay), u (unit key) and b (removal rate times unit key) come per row and key channel from k_chan_delta_gates.
// grid (rows, heads): a workgroup per head of a row.  The bottleneck's activations tanh(lr) in LDS, then a thread per key channel:
// decay = exp(-mult * sigmoid(w2[c] . tanh(lr) + w0[c])), u = k / sqrt(sum k^2 + l2_eps), b = sigmoid(a) * u.
// rank 0: lr holds the sigmoid's argument itself, [heads * dim] per row (larger steps form it as a matrix product).
__global__ void __launch_bounds__(256) k_chan_delta_gates(const float *lr, size_t ldl, int rank, const bf16_t *__restrict__ w2, const bf16_t *__restrict__ w0,
                                                          float mult, const float *__restrict__ a, size_t lda, const float *__restrict__ k, size_t ldk, int H, int D,
                                                          float l2_eps, float *decay, float *__restrict__ unit, float *__restrict__ removal, int vec)      // (rank 0: decay may be lr itself)
{
    extern __shared__ float th[];          // [rank]
    __shared__ float red[17];
    const int t = blockIdx.x, h = blockIdx.y;
    for (int i = threadIdx.x; i < rank; i += blockDim.x) th[i] = tanhf(lr[(size_t)t * ldl + i]);
    const size_t HD = (size_t)H * D;
    const float *kr = k + (size_t)t * ldk + (size_t)h * D;
    float s = 0.0f;
    for (int c = threadIdx.x; c < D; c += blockDim.x) s = fmaf(kr[c], kr[c], s);
    const float rinv = 1.0f / sqrtf(block_sum(s, red) + l2_eps);          // (its barriers also publish th)
    for (int c = threadIdx.x; c < D; c += blockDim.x) {
        const size_t hc = (size_t)h * D + c;
        float z;
        if (rank > 0) {
            const bf16_t *wr = w2 + hc * (size_t)rank;
            float z0 = w0 ? bf2f(w0[hc]) : 0.0f, z1 = 0.0f;
            int i = 0;
            if (vec) {          // rows of whole 16-byte pieces
                for (; i + 8 <= rank; i += 8) {
                    const uint4 wv = *reinterpret_cast<const uint4 *>(wr + i);
                    z0 = fmaf(__uint_as_float(wv.x << 16), th[i], z0); z1 = fmaf(__uint_as_float(wv.x & 0xFFFF0000u), th[i + 1], z1);
                    z0 = fmaf(__uint_as_float(wv.y << 16), th[i + 2], z0); z1 = fmaf(__uint_as_float(wv.y & 0xFFFF0000u), th[i + 3], z1);
                    z0 = fmaf(__uint_as_float(wv.z << 16), th[i + 4], z0); z1 = fmaf(__uint_as_float(wv.z & 0xFFFF0000u), th[i + 5], z1);
                    z0 = fmaf(__uint_as_float(wv.w << 16), th[i + 6], z0); z1 = fmaf(__uint_as_float(wv.w & 0xFFFF0000u), th[i + 7], z1);
                }
            }
            for (; i + 1 < rank; i += 2) { z0 = fmaf(bf2f(wr[i]), th[i], z0); z1 = fmaf(bf2f(wr[i + 1]), th[i + 1], z1); }
            if (i < rank) z0 = fmaf(bf2f(wr[i]), th[i], z0);
            z = z0 + z1;
        } else z = lr[(size_t)t * ldl + hc];
        const float u = kr[c] * rinv;
        decay[(size_t)t * HD + hc] = expf(-mult * sigmoid_f(z));
        unit[(size_t)t * HD + hc] = u;
        removal[(size_t)t * HD + hc] = sigmoid_f(a[(size_t)t * lda + hc]) * u;
    }
}

// x[t][c] = tanh(x[t][c]) in place over a column range of the rows
__global__ void __launch_bounds__(256) k_tanh_cols(float *__restrict__ x, size_t ldx, int cols)
{
    float *xr = x + (size_t)blockIdx.x * ldx;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) xr[c] = tanhf(xr[c]);
}

struct ChanScanArgs {
    const float *q, *k, *v; size_t ldq, ldk, ldv;
    const float *w, *u, *b; size_t ldg;
    int heads, dk, dv;
    const SeqDesc *seqs; float *const *slot_base; size_t state_off;
    float *out; size_t ldo;
};

// any dk <= 64 * SCAN_DKL: grid (sequences * heads, ceil(dv / 64)), one wave; a lane owns a column of S in LDS ([dk][64])
__global__ void __launch_bounds__(64) k_state_scan_chan(ChanScanArgs P)
{
    extern __shared__ float sm[];
    const int dk = P.dk;
    float *S = sm, *qs = sm + (size_t)dk * 64, *ks = qs + dk, *ws = ks + dk, *us = ws + dk, *bs = us + dk;
    const int seq = blockIdx.x / P.heads, h = blockIdx.x % P.heads;
    const int lane = threadIdx.x, j = blockIdx.y * 64 + lane;
    const bool live = j < P.dv;
    const int jc = live ? j : P.dv - 1;
    const SeqDesc sd = P.seqs[seq];
    float *state = P.slot_base[sd.slot] + P.state_off + (size_t)h * dk * P.dv;
    if (sd.pos0 > 0) for (int i = 0; i < dk; i++) S[i * 64 + lane] = state[(size_t)i * P.dv + jc];
    else for (int i = 0; i < dk; i++) S[i * 64 + lane] = 0.0f;
    float qr[SCAN_DKL], kr[SCAN_DKL], wr[SCAN_DKL], ur[SCAN_DKL], br[SCAN_DKL], vr = 0.0f;
    auto request = [&](int t) {
        const size_t row = (size_t)(sd.row0 + t);
#pragma unroll
        for (int e = 0; e < SCAN_DKL; e++) {
            const int i = lane + 64 * e;
            if (i < dk) {
                const size_t hc = (size_t)h * dk + i;
                qr[e] = P.q[row * P.ldq + hc]; kr[e] = P.k[row * P.ldk + hc];
                wr[e] = P.w[row * P.ldg + hc]; ur[e] = P.u[row * P.ldg + hc]; br[e] = P.b[row * P.ldg + hc];
            }
        }
        vr = P.v[row * P.ldv + (size_t)h * P.dv + jc];
    };
    if (sd.n > 0) request(0);
    for (int t = 0; t < sd.n; t++) {
        __syncthreads();          // the previous token's reads of the staged vectors are done
#pragma unroll
        for (int e = 0; e < SCAN_DKL; e++) { const int i = lane + 64 * e; if (i < dk) { qs[i] = qr[e]; ks[i] = kr[e]; ws[i] = wr[e]; us[i] = ur[e]; bs[i] = br[e]; } }
        const float vt = vr;
        __syncthreads();
        if (t + 1 < sd.n) request(t + 1);
        float sa = 0.0f, o = 0.0f;
        for (int i = 0; i < dk; i++) sa = fmaf(us[i], S[i * 64 + lane], sa);
        for (int i = 0; i < dk; i++) {
            const float s = fmaf(ks[i], vt, fmaf(ws[i], S[i * 64 + lane], -bs[i] * sa));
            S[i * 64 + lane] = s;
            o = fmaf(s, qs[i], o);
        }
        if (live) P.out[(size_t)(sd.row0 + t) * P.ldo + (size_t)h * P.dv + j] = o;
    }
    if (live) for (int i = 0; i < dk; i++) state[(size_t)i * P.dv + j] = S[i * 64 + lane];
}

// key sizes 16 / 32 / 48 / 64 / 96 / 128: the state in registers, LPC lanes per column (as k_state_scan_reg; sixteen lanes from 128 key channels on, so
// that a lane walks eight rows of its column per token and a head's columns are spread over twice as many waves), token groups of SCAN_TB staged in LDS
template <int DK, int LPC>
__global__ void __launch_bounds__(64) k_state_scan_chan_reg(ChanScanArgs P)
{
    constexpr int DKQ = DK / LPC, CPW = 64 / LPC;
    __shared__ __attribute__((aligned(16))) float qs[2][SCAN_TB][DK], ks[2][SCAN_TB][DK], ws[2][SCAN_TB][DK], us[2][SCAN_TB][DK], bs[2][SCAN_TB][DK];
    const int seq = blockIdx.x / P.heads, h = blockIdx.x % P.heads;
    const int lane = threadIdx.x, rg = lane & (LPC - 1), j = blockIdx.y * CPW + lane / LPC;
    const bool live = j < P.dv;
    const int jc = live ? j : P.dv - 1;
    const SeqDesc sd = P.seqs[seq];
    float *state = P.slot_base[sd.slot] + P.state_off + ((size_t)h * DK + (size_t)rg * DKQ) * P.dv;
    float S[DKQ];
    if (sd.pos0 > 0) {
#pragma unroll
        for (int e = 0; e < DKQ; e++) S[e] = state[(size_t)e * P.dv + jc];
    } else {
#pragma unroll
        for (int e = 0; e < DKQ; e++) S[e] = 0.0f;
    }
    constexpr int PER = SCAN_TB * DK / 64;
    float qr[PER], kr[PER], wr[PER], ur[PER], br[PER], vnext[SCAN_TB], vcur[SCAN_TB];
    auto request = [&](int t0) {
#pragma unroll
        for (int x = 0; x < PER; x++) {
            const int e = lane + 64 * x, tt = e / DK, i = e % DK;
            const size_t row = (size_t)(sd.row0 + min(t0 + tt, sd.n - 1)), hc = (size_t)h * DK + i;
            qr[x] = P.q[row * P.ldq + hc]; kr[x] = P.k[row * P.ldk + hc];
            wr[x] = P.w[row * P.ldg + hc]; ur[x] = P.u[row * P.ldg + hc]; br[x] = P.b[row * P.ldg + hc];
        }
#pragma unroll
        for (int tt = 0; tt < SCAN_TB; tt++) {
            const size_t row = (size_t)(sd.row0 + min(t0 + tt, sd.n - 1));
            vnext[tt] = P.v[row * P.ldv + (size_t)h * P.dv + jc];
        }
    };
    auto publish = [&](int buf) {
#pragma unroll
        for (int x = 0; x < PER; x++) {
            const int e = lane + 64 * x, tt = e / DK, i = e % DK;
            // channel i = rg DKQ + e lies at [e / 4][rg][e % 4]: the lanes' 16-byte reads of one step are consecutive pieces (no bank is asked twice)
            const int pi = ((i % DKQ) / 4) * (LPC * 4) + (i / DKQ) * 4 + (i % 4);
            qs[buf][tt][pi] = qr[x]; ks[buf][tt][pi] = kr[x]; ws[buf][tt][pi] = wr[x]; us[buf][tt][pi] = ur[x]; bs[buf][tt][pi] = br[x];
        }
#pragma unroll
        for (int tt = 0; tt < SCAN_TB; tt++) vcur[tt] = vnext[tt];
    };
    if (sd.n > 0) { request(0); publish(0); }
    __syncthreads();
    for (int t0 = 0, buf = 0; t0 < sd.n; t0 += SCAN_TB, buf ^= 1) {
        const bool more = t0 + SCAN_TB < sd.n;
        if (more) request(t0 + SCAN_TB);
        const int cnt = min(SCAN_TB, sd.n - t0);
        // one token.  What does not depend on the state (k v, -b) is formed ahead; from the column's sum sa to the new state are two dependent operations
        auto token = [&](int tt) {
            const float vt = vcur[tt];
            float kv[DKQ], qq[DKQ], ww[DKQ], uu[DKQ], nb[DKQ];
#pragma unroll
            for (int e4 = 0; e4 < DKQ; e4 += 4) {
                const float4 k4 = *reinterpret_cast<const float4 *>(&ks[buf][tt][e4 * LPC + rg * 4]), q4 = *reinterpret_cast<const float4 *>(&qs[buf][tt][e4 * LPC + rg * 4]);
                const float4 w4 = *reinterpret_cast<const float4 *>(&ws[buf][tt][e4 * LPC + rg * 4]), u4 = *reinterpret_cast<const float4 *>(&us[buf][tt][e4 * LPC + rg * 4]);
                const float4 b4 = *reinterpret_cast<const float4 *>(&bs[buf][tt][e4 * LPC + rg * 4]);
                kv[e4] = k4.x * vt; kv[e4 + 1] = k4.y * vt; kv[e4 + 2] = k4.z * vt; kv[e4 + 3] = k4.w * vt;
                qq[e4] = q4.x; qq[e4 + 1] = q4.y; qq[e4 + 2] = q4.z; qq[e4 + 3] = q4.w;
                ww[e4] = w4.x; ww[e4 + 1] = w4.y; ww[e4 + 2] = w4.z; ww[e4 + 3] = w4.w;
                uu[e4] = u4.x; uu[e4 + 1] = u4.y; uu[e4 + 2] = u4.z; uu[e4 + 3] = u4.w;
                nb[e4] = -b4.x; nb[e4 + 1] = -b4.y; nb[e4 + 2] = -b4.z; nb[e4 + 3] = -b4.w;
            }
            float r0 = 0.0f, r1 = 0.0f;
#pragma unroll
            for (int e = 0; e < DKQ; e += 2) { r0 = fmaf(S[e], uu[e], r0); r1 = fmaf(S[e + 1], uu[e + 1], r1); }
            const float sa = LPC == 16 ? hex_sum(r0 + r1) : (LPC == 8 ? oct_sum(r0 + r1) : quad_sum(r0 + r1));
            float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
            for (int e = 0; e < DKQ; e += 2) {
                S[e] = fmaf(ww[e], S[e], fmaf(nb[e], sa, kv[e])); o0 = fmaf(S[e], qq[e], o0);
                S[e + 1] = fmaf(ww[e + 1], S[e + 1], fmaf(nb[e + 1], sa, kv[e + 1])); o1 = fmaf(S[e + 1], qq[e + 1], o1);
            }
            const float o = LPC == 16 ? hex_sum(o0 + o1) : (LPC == 8 ? oct_sum(o0 + o1) : quad_sum(o0 + o1));
            if (live && rg == 0) P.out[(size_t)(sd.row0 + t0 + tt) * P.ldo + (size_t)h * P.dv + j] = o;
        };
        if (cnt == SCAN_TB) {      // a whole group: straight-line code, so that a token's read-out overlaps the next token's chain
#pragma unroll
            for (int tt = 0; tt < SCAN_TB; tt++) token(tt);
        } else {
#pragma unroll
            for (int tt = 0; tt < SCAN_TB; tt++) if (tt < cnt) token(tt);
        }
        if (more) publish(buf ^ 1);
        __syncthreads();
    }
    if (live) {
#pragma unroll
        for (int e = 0; e < DKQ; e++) state[(size_t)e * P.dv + j] = S[e];
    }
}

// y[t][c] = o[t][c] / sqrt(mean_group(o^2) + eps) * w[c % wlen] * act(gate[t][c]); one workgroup per row, a wave per group
__global__ void __launch_bounds__(256) k_gated_groupnorm(const float *__restrict__ o, size_t ldo, int C, int group, const bf16_t *__restrict__ w, int wlen,
                                                         const float *__restrict__ gate, size_t ldg, int gate_act, float eps, float *__restrict__ y,
                                                         size_t ldy)
{
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float *orow = o + (size_t)t * ldo, *grow = gate + (size_t)t * ldg;
    float *yrow = y + (size_t)t * ldy;
    if (C / group < nw) {          // fewer groups than waves (one norm over all heads): the whole workgroup works on each group
        __shared__ float red[17];
        for (int gi = 0; gi < C / group; gi++) {
            float s = 0.0f;
            for (int e = threadIdx.x; e < group; e += blockDim.x) { const float v = orow[gi * group + e]; s = fmaf(v, v, s); }
            const float r = 1.0f / sqrtf(block_sum(s, red) / (float)group + eps);
            for (int e = threadIdx.x; e < group; e += blockDim.x) {
                const int c = gi * group + e;
                const float gv = grow[c];
                const float ga = gate_act == 0 ? sigmoid_f(gv) : silu_exact(gv);
                yrow[c] = orow[c] * r * bf2f(w[c % wlen]) * ga;
            }
        }
        return;
    }
    for (int gi = wave; gi < C / group; gi += nw) {
        float s = 0.0f;
        for (int e = lane; e < group; e += 64) { const float v = orow[gi * group + e]; s = fmaf(v, v, s); }
        s = wave_sum(s);
        const float r = 1.0f / sqrtf(s / (float)group + eps);
        for (int e = lane; e < group; e += 64) {
            const int c = gi * group + e;
            const float gv = grow[c];
            const float ga = gate_act == 0 ? sigmoid_f(gv) : silu_exact(gv);
            yrow[c] = orow[c] * r * bf2f(w[c % wlen]) * ga;
        }
    }
}

} // namespace

extern "C" {

int ifa_shortconv_silu_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *w_bf16, const void *seqs_dev, const int *row_seq_dev,
                           size_t rows, void *const *slot_base_dev, size_t state_off, int norm_cols, int group_dim, float l2_eps, int scale_cols,
                           float scale, void *y_f32, size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && w_bf16 && seqs_dev && row_seq_dev && slot_base_dev && y_f32, "ifa_shortconv_silu_f32: null pointer");
    IFA_REQUIRE(channels > 0 && taps >= 1 && taps <= 64 && rows > 0 && ldx >= (size_t)channels && ldy >= (size_t)channels, "ifa_shortconv_silu_f32: bad shape");
    IFA_REQUIRE(norm_cols >= 0 && norm_cols <= channels && scale_cols >= 0 && scale_cols <= channels && (norm_cols == 0 || (group_dim > 0 && norm_cols % group_dim == 0)),
                "ifa_shortconv_silu_f32: bad norm groups");
    // a row's channels go to several workgroups in slices of whole norm groups (~512 channels: steps of a few rows would otherwise
    // leave the convolution to one workgroup)
    const int gd = norm_cols > 0 ? group_dim : 1;
    const int slice = std::min(channels, gd * std::max(1, (512 + gd - 1) / gd));
    IFA_REQUIRE((size_t)slice * 4 <= 64 * 1024, "ifa_shortconv_silu_f32: norm groups of %d channels do not fit the LDS", group_dim);
    hipLaunchKernelGGL(k_shortconv_silu, dim3((unsigned)rows, ifa_cdiv((size_t)channels, (size_t)slice)), dim3(256), (size_t)slice * 4, ifa_s(stream),
                       (const float *)x_f32, ldx, channels, taps, (const bf16_t *)w_bf16, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev,
                       state_off, norm_cols, group_dim, l2_eps, scale_cols, scale, (float *)y_f32, ldy, slice);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_shortconv_residual_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *w_bf16, const void *seqs_dev, const int *row_seq_dev,
                               size_t rows, void *const *slot_base_dev, size_t state_off, void *y_f32, size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && w_bf16 && seqs_dev && row_seq_dev && slot_base_dev && y_f32 && x_f32 != y_f32, "ifa_shortconv_residual_f32: null pointer or y = x");
    IFA_REQUIRE(channels > 0 && taps >= 1 && taps <= 64 && rows > 0 && ldx >= (size_t)channels && ldy >= (size_t)channels, "ifa_shortconv_residual_f32: bad shape");
    hipLaunchKernelGGL(k_shortconv_residual, dim3((unsigned)rows, std::min(8u, ifa_cdiv((size_t)channels, 256))), dim3(256), 0, ifa_s(stream), (const float *)x_f32, ldx,
                       channels, taps, (const bf16_t *)w_bf16, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, state_off, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_norm_add_conv_rows_f32(void *x_f32, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *norm_w_bf16, int groups, float eps,
                               void *stack_f32, size_t plane_stride, int count, const void *depth_w_bf16, const void *conv_w_bf16, int taps,
                               const void *seqs_dev, int n_seqs, const int *row_seq_dev, void *const *slot_base_dev, size_t state_off, void *h_f32,
                               ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && rows > 0 && rows <= 64 && cols > 0 && rows * cols < (1u << 30), "ifa_norm_add_conv_rows_f32: bad shape (%zu rows: at most 64)", rows);
    IFA_REQUIRE(!m_f32 || (groups >= 1 && cols % (size_t)groups == 0 && ldm >= cols), "ifa_norm_add_conv_rows_f32: bad norm");
    IFA_REQUIRE(!stack_f32 || (depth_w_bf16 && count >= 1 && plane_stride >= rows * cols), "ifa_norm_add_conv_rows_f32: bad depth average");
    IFA_REQUIRE(!conv_w_bf16 || (taps >= 1 && taps <= 64 && seqs_dev && n_seqs > 0 && row_seq_dev && slot_base_dev && h_f32 && h_f32 != x_f32),
                "ifa_norm_add_conv_rows_f32: bad convolution");
    // a workgroup per norm part; without a norm the channels are shared out the same way (up to 64 parts that divide the row)
    int parts = groups;
    if (!m_f32) { parts = 1; while (parts < 64 && cols % (size_t)(parts * 2) == 0 && cols / (size_t)(parts * 2) >= 64) parts *= 2; }
    hipLaunchKernelGGL(k_norm_add_conv_rows, dim3((unsigned)parts), dim3(256), 0, ifa_s(stream), (float *)x_f32, (int)rows, (int)cols, (const float *)m_f32, ldm,
                       (const bf16_t *)norm_w_bf16, parts, eps, (float *)stack_f32, plane_stride, count, (const bf16_t *)depth_w_bf16, (const bf16_t *)conv_w_bf16, taps,
                       (const SeqDesc *)seqs_dev, n_seqs, row_seq_dev, (float *const *)slot_base_dev, state_off, (float *)h_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_shortconv_tail_f32(const void *x_f32, size_t ldx, int channels, int taps, const void *seqs_dev, int n_seqs, void *const *slot_base_dev,
                           size_t state_off, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && seqs_dev && slot_base_dev, "ifa_shortconv_tail_f32: null pointer");
    IFA_REQUIRE(channels > 0 && taps >= 1 && n_seqs > 0 && ldx >= (size_t)channels, "ifa_shortconv_tail_f32: bad shape");
    if (taps == 1) return IFA_OK;
    hipLaunchKernelGGL(k_shortconv_tail, dim3((unsigned)n_seqs), dim3(256), 0, ifa_s(stream), (const float *)x_f32, ldx, channels, taps,
                       (const SeqDesc *)seqs_dev, (float *const *)slot_base_dev, state_off);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_delta_gates_f32(const void *b_f32, size_t ldb, const void *a_f32, size_t lda, int heads, size_t rows, const void *a_log_bf16,
                        const void *dt_bias_bf16, void *beta_f32, void *decay_f32, ifa_stream stream)
{
    IFA_REQUIRE(b_f32 && a_f32 && a_log_bf16 && dt_bias_bf16 && beta_f32 && decay_f32, "ifa_delta_gates_f32: null pointer");
    IFA_REQUIRE(heads > 0 && rows > 0 && ldb >= (size_t)heads && lda >= (size_t)heads, "ifa_delta_gates_f32: bad shape");
    hipLaunchKernelGGL(k_delta_gates, dim3(ifa_cdiv(rows * heads, 256)), dim3(256), 0, ifa_s(stream), (const float *)b_f32, ldb, (const float *)a_f32, lda,
                       heads, (int)rows, (const bf16_t *)a_log_bf16, (const bf16_t *)dt_bias_bf16, (float *)beta_f32, (float *)decay_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_state_scan_f32(int kind, int in_act, const void *q_f32, size_t ldq, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int heads, int qk_heads,
                       int dk, int dv, const void *decay_head_f32, const void *decay_row_f32, const void *beta_row_f32, const void *seqs_dev, int n_seqs,
                       void *const *slot_base_dev, size_t state_off, void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && k_f32 && v_f32 && seqs_dev && slot_base_dev && out_f32, "ifa_state_scan_f32: null pointer");
    IFA_REQUIRE(kind == 0 || kind == 1, "ifa_state_scan_f32: kind %d", kind);
    IFA_REQUIRE(heads > 0 && qk_heads > 0 && heads % qk_heads == 0 && dk > 0 && dv > 0 && n_seqs > 0, "ifa_state_scan_f32: bad shape");
    IFA_REQUIRE(dk <= 64 * SCAN_DKL, "ifa_state_scan_f32: key size %d above %d", dk, 64 * SCAN_DKL);
    IFA_REQUIRE(kind == 0 ? decay_head_f32 != nullptr : (decay_row_f32 && beta_row_f32), "ifa_state_scan_f32: the gates of kind %d are missing", kind);
    ScanArgs P;
    P.q = (const float *)q_f32; P.k = (const float *)k_f32; P.v = (const float *)v_f32; P.ldq = ldq; P.ldk = ldk; P.ldv = ldv;
    P.heads = heads; P.qk_heads = qk_heads; P.dk = dk; P.dv = dv; P.in_act = in_act ? 1 : 0;
    P.decay_head = (const float *)decay_head_f32; P.decay_row = (const float *)decay_row_f32; P.beta_row = (const float *)beta_row_f32;
    P.seqs = (const SeqDesc *)seqs_dev; P.slot_base = (float *const *)slot_base_dev; P.state_off = state_off;
    P.out = (float *)out_f32; P.ldo = ldo;
    const size_t smem = ((size_t)dk * 64 + 2 * (size_t)dk) * 4;
    const dim3 grid((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 64));
    // four lanes per column (16 columns per wave); key sizes from 64 on: eight lanes per column (8 columns per wave)
    const dim3 grid16((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 16)), grid8((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 8));
#define IFA_SCAN_REG(DKV) \
    if (dk == DKV) { \
        if (DKV >= 64) { \
            if (kind == 0) hipLaunchKernelGGL((k_state_scan_reg<0, DKV, 8>), grid8, dim3(64), 0, ifa_s(stream), P); \
            else hipLaunchKernelGGL((k_state_scan_reg<1, DKV, 8>), grid8, dim3(64), 0, ifa_s(stream), P); \
        } else if (kind == 0) hipLaunchKernelGGL((k_state_scan_reg<0, DKV, 4>), grid16, dim3(64), 0, ifa_s(stream), P); \
        else hipLaunchKernelGGL((k_state_scan_reg<1, DKV, 4>), grid16, dim3(64), 0, ifa_s(stream), P); \
        IFA_LAUNCH_CHECK(); \
        return IFA_OK; \
    }
    IFA_SCAN_REG(16) IFA_SCAN_REG(32) IFA_SCAN_REG(64) IFA_SCAN_REG(128)
#undef IFA_SCAN_REG
    if (kind == 0) {
        IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_state_scan<0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(k_state_scan<0>, grid, dim3(64), smem, ifa_s(stream), P);
    } else {
        IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_state_scan<1>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        hipLaunchKernelGGL(k_state_scan<1>, grid, dim3(64), smem, ifa_s(stream), P);
    }
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_chan_delta_gates_f32(const void *lr_f32, size_t ldl, int rank, const void *w2_bf16, const void *w0_bf16, float decay_mult, const void *a_f32, size_t lda,
                             const void *k_f32, size_t ldk, int heads, int dim, float l2_eps, size_t rows, void *decay_f32, void *unit_f32, void *removal_f32,
                             ifa_stream stream)
{
    IFA_REQUIRE(lr_f32 && (rank == 0 || w2_bf16) && a_f32 && k_f32 && decay_f32 && unit_f32 && removal_f32, "ifa_chan_delta_gates_f32: null pointer");
    const size_t HD = (size_t)heads * dim;
    IFA_REQUIRE(heads > 0 && dim > 0 && rows > 0 && rank >= 0 && rank <= 8192 && ldl >= (rank > 0 ? (size_t)rank : HD) && lda >= HD && ldk >= HD,
                "ifa_chan_delta_gates_f32: bad shape");
    IFA_REQUIRE(heads < 65536, "ifa_chan_delta_gates_f32: %d heads", heads);
    const int vec = (rank % 8 == 0 && ((uintptr_t)w2_bf16 & 15) == 0) ? 1 : 0;
    hipLaunchKernelGGL(k_chan_delta_gates, dim3((unsigned)rows, (unsigned)heads), dim3(dim <= 64 ? 64 : (dim <= 128 ? 128 : 256)), (size_t)rank * 4, ifa_s(stream),
                       (const float *)lr_f32, ldl, rank, (const bf16_t *)w2_bf16, (const bf16_t *)w0_bf16, decay_mult, (const float *)a_f32, lda, (const float *)k_f32, ldk,
                       heads, dim, l2_eps, (float *)decay_f32, (float *)unit_f32, (float *)removal_f32, vec);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_tanh_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && rows > 0 && rows < (1u << 31) && cols > 0 && ldx >= cols, "ifa_tanh_f32: bad arguments");
    hipLaunchKernelGGL(k_tanh_cols, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (float *)x_f32, ldx, (int)cols);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_state_scan_chan_f32(const void *q_f32, size_t ldq, const void *k_f32, size_t ldk, const void *v_f32, size_t ldv, int heads, int dk, int dv,
                            const void *decay_f32, const void *unit_f32, const void *removal_f32, size_t ldg, const void *seqs_dev, int n_seqs,
                            void *const *slot_base_dev, size_t state_off, void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(q_f32 && k_f32 && v_f32 && decay_f32 && unit_f32 && removal_f32 && seqs_dev && slot_base_dev && out_f32, "ifa_state_scan_chan_f32: null pointer");
    IFA_REQUIRE(heads > 0 && dk > 0 && dv > 0 && n_seqs > 0 && dk <= 64 * SCAN_DKL, "ifa_state_scan_chan_f32: bad shape (key size %d: at most %d)", dk, 64 * SCAN_DKL);
    const size_t HK = (size_t)heads * dk, HV = (size_t)heads * dv;
    IFA_REQUIRE(ldq >= HK && ldk >= HK && ldg >= HK && ldv >= HV && ldo >= HV, "ifa_state_scan_chan_f32: row strides too small");
    ChanScanArgs P;
    P.q = (const float *)q_f32; P.k = (const float *)k_f32; P.v = (const float *)v_f32; P.ldq = ldq; P.ldk = ldk; P.ldv = ldv;
    P.w = (const float *)decay_f32; P.u = (const float *)unit_f32; P.b = (const float *)removal_f32; P.ldg = ldg;
    P.heads = heads; P.dk = dk; P.dv = dv;
    P.seqs = (const SeqDesc *)seqs_dev; P.slot_base = (float *const *)slot_base_dev; P.state_off = state_off;
    P.out = (float *)out_f32; P.ldo = ldo;
    const dim3 grid16((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 16)), grid8((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 8));
    const dim3 grid4((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 4));
#define IFA_CSCAN(DKV, L, G) if (dk == DKV) { hipLaunchKernelGGL((k_state_scan_chan_reg<DKV, L>), G, dim3(64), 0, ifa_s(stream), P); IFA_LAUNCH_CHECK(); return IFA_OK; }
    IFA_CSCAN(16, 4, grid16) IFA_CSCAN(32, 4, grid16) IFA_CSCAN(48, 4, grid16) IFA_CSCAN(64, 8, grid8) IFA_CSCAN(96, 8, grid8) IFA_CSCAN(128, 16, grid4)
#undef IFA_CSCAN
    const size_t smem = ((size_t)dk * 64 + 5 * (size_t)dk) * 4;
    IFA_HIP_CHECK(hipFuncSetAttribute((const void *)k_state_scan_chan, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    hipLaunchKernelGGL(k_state_scan_chan, dim3((unsigned)(n_seqs * heads), ifa_cdiv((size_t)dv, 64)), dim3(64), smem, ifa_s(stream), P);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_gated_groupnorm_f32(const void *o_f32, size_t ldo, size_t rows, int channels, int group, const void *w_bf16, int wlen, const void *gate_f32,
                            size_t ldg, int gate_act, float eps, void *y_f32, size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(o_f32 && w_bf16 && gate_f32 && y_f32, "ifa_gated_groupnorm_f32: null pointer");
    IFA_REQUIRE(rows > 0 && channels > 0 && group > 0 && channels % group == 0 && wlen > 0 && (gate_act == 0 || gate_act == 1), "ifa_gated_groupnorm_f32: bad arguments");
    hipLaunchKernelGGL(k_gated_groupnorm, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const float *)o_f32, ldo, channels, group,
                       (const bf16_t *)w_bf16, wlen, (const float *)gate_f32, ldg, gate_act, eps, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

} // extern "C"
