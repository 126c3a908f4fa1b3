// ifa_ops_f32.hip -- element-wise and row ops on 32-bit activations with bfloat16 parameters: embedding rows with a sinusoidal
// position vector, layer / RMS norm, gated activations, greedy argmax, and the conversions the F16 interfaces need.
#include <algorithm>
#include "ifa_host.h"
#include "ifa_f32_common.h"

using namespace ifa32;

namespace {

// x[t][c] = embed[token_t][c] + pe(pos_t)[c];  pe[2i] = sin(p w_i), pe[2i + 1] = cos(p w_i), w_i = base^(-2i / width).
// The angle of position p reaches hundreds of radians where one fp32 ulp is already 1e-4: it is formed in double.
__global__ void __launch_bounds__(256) k_embed_sinpos(const bf16_t *__restrict__ embed, int vocab, int width, const int *__restrict__ tokens,
                                                      const int *__restrict__ positions, double base_log, float *__restrict__ x)
{
    const int t = blockIdx.x;
    const int tok = min(max(tokens[t], 0), vocab - 1);
    const double p = (double)positions[t];
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        const int i2 = c & ~1;
        const double w = exp(-(double)i2 / (double)width * base_log);
        const double a = p * w;
        const float pe = (float)((c & 1) ? cos(a) : sin(a));
        x[(size_t)t * width + c] = bf2f(embed[(size_t)tok * width + c]) + pe;
    }
}

// kind 0: y = x / sqrt(mean(x^2) + eps) * w;  kind 1: y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w.  w may be null.
__global__ void __launch_bounds__(256) k_norm_f32(int kind, const float *__restrict__ x, size_t ldx, int cols, const bf16_t *__restrict__ w, float eps,
                                                  float *__restrict__ y, size_t ldy)
{
    __shared__ float red[17];
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    float mean = 0.0f;
    if (kind == 1) {
        float s = 0.0f;
        for (int c = threadIdx.x; c < cols; c += blockDim.x) s += xr[c];
        mean = block_sum(s, red) / (float)cols;
    }
    float q = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) { const float d = xr[c] - mean; q += d * d; }
    const float rinv = 1.0f / sqrtf(block_sum(q, red) / (float)cols + eps);
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = (xr[c] - mean) * rinv;
        yr[c] = w ? v * bf2f(w[c]) : v;
    }
}

// x[t][c] = embed[token_t][c], no position vector
__global__ void __launch_bounds__(256) k_embed_rows(const bf16_t *__restrict__ embed, int vocab, int width, const int *__restrict__ tokens, float *__restrict__ x)
{
    const int t = blockIdx.x;
    const int tok = min(max(tokens[t], 0), vocab - 1);
    for (int c = threadIdx.x; c < width; c += blockDim.x) x[(size_t)t * width + c] = bf2f(embed[(size_t)tok * width + c]);
}

// RMS norm in `groups` consecutive parts of a row, a wave per part at a time: y (+)= x / sqrt(mean_part(x^2) + eps) * w
__global__ void __launch_bounds__(256) k_group_rmsnorm(const float *__restrict__ x, size_t ldx, int cols, int groups, const bf16_t *__restrict__ w, float eps,
                                                       int accumulate, float *__restrict__ y, size_t ldy)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    const int gs = cols / groups;
    for (int g = wave; g < groups; g += nw) {
        float q = 0.0f;
        for (int c = lane; c < gs; c += 64) { const float v = xr[g * gs + c]; q = fmaf(v, v, q); }
        const float rinv = 1.0f / sqrtf(wave_sum(q) / (float)gs + eps);
        for (int c = lane; c < gs; c += 64) {
            const int cc = g * gs + c;
            float v = xr[cc] * rinv;
            if (w) v *= bf2f(w[cc]);
            yr[cc] = accumulate ? yr[cc] + v : v;
        }
    }
}

// x[t] = embed[token_t] + pair[row_t]; row_t = (prev_t * mul_prev + token_t * mul_cur) mod buckets, or `buckets` at position 0.  The
// workgroup of a sequence's first row is the only one that reads the token the slot holds, and it leaves the sequence's last token
// of this step there: no other workgroup touches that cell.
__global__ void __launch_bounds__(256) k_embed_pair(const bf16_t *__restrict__ embed, int vocab, int width, const bf16_t *__restrict__ pair, int buckets,
                                                    int mul_prev, int mul_cur, const int *__restrict__ tokens, const SeqDesc *__restrict__ seqs,
                                                    const int *__restrict__ row_seq, float *const *__restrict__ slot_base, size_t state_off,
                                                    float *__restrict__ x, float embed_scale, float *__restrict__ x_copy)
{
    const int t = blockIdx.x;
    const SeqDesc sd = seqs[row_seq[t]];
    const int tok = min(max(tokens[t], 0), vocab - 1);
    int *cell = reinterpret_cast<int *>(slot_base[sd.slot] + state_off);
    int prow = buckets;
    if (pair) {
        const int pos = sd.pos0 + t - sd.row0;
        if (pos > 0) {
            const int prev = t > sd.row0 ? tokens[t - 1] : *cell;
            prow = (int)(((long long)prev * mul_prev + (long long)tok * mul_cur) % (long long)buckets);
            if (prow < 0) prow += buckets;
        }
    }
    __syncthreads();      // (the read of the cell above is done in every thread before thread 0 rewrites it)
    if (t == sd.row0 && threadIdx.x == 0) *cell = tokens[sd.row0 + sd.n - 1];
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float v = bf2f(embed[(size_t)tok * width + c]) * embed_scale;
        if (pair) v += bf2f(pair[(size_t)prow * width + c]);
        x[(size_t)t * width + c] = v;
        if (x_copy) x_copy[(size_t)t * width + c] = v;
    }
}

// Dynamic Tanh: y = tanh(alpha x) w + b, element by element (alpha: one bfloat16 value)
__global__ void __launch_bounds__(256) k_dyt(const float *__restrict__ x, size_t ldx, int cols, const bf16_t *__restrict__ alpha, const bf16_t *__restrict__ w,
                                             const bf16_t *__restrict__ b, float *__restrict__ y, size_t ldy)
{
    const float a = bf2f(alpha[0]);
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < cols; c += gridDim.y * blockDim.x) yr[c] = fmaf(tanhf(a * xr[c]), bf2f(w[c]), bf2f(b[c]));
}

// x += m + vec, then h = tanh(alpha x) w + b: the residual update behind a sub-layer (or the start of a looped pass) and the norm in front of the next one
__global__ void __launch_bounds__(256) k_add_dyt(float *__restrict__ x, size_t ldx, int cols, const float *__restrict__ m, size_t ldm, const bf16_t *__restrict__ vec,
                                                 const bf16_t *__restrict__ alpha, const bf16_t *__restrict__ w, const bf16_t *__restrict__ b, float *__restrict__ h, size_t ldh)
{
    const float a = w ? bf2f(alpha[0]) : 0.0f;
    float *xr = x + (size_t)blockIdx.x * ldx;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < cols; c += gridDim.y * blockDim.x) {
        float v = xr[c];
        if (m || vec) {
            if (m) v += m[(size_t)blockIdx.x * ldm + c];
            if (vec) v += bf2f(vec[c]);
            xr[c] = v;
        }
        if (w) h[(size_t)blockIdx.x * ldh + c] = fmaf(tanhf(a * v), bf2f(w[c]), bf2f(b[c]));
    }
}

// x[t][c] += add[t][c] + vec[c] (either may be absent)
__global__ void __launch_bounds__(256) k_add_rows_vec(float *__restrict__ x, size_t ldx, int cols, const float *__restrict__ add, size_t lda,
                                                      const bf16_t *__restrict__ vec)
{
    float *xr = x + (size_t)blockIdx.x * ldx;
    for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < cols; c += gridDim.y * blockDim.x) {
        float v = xr[c];
        if (add) v += add[(size_t)blockIdx.x * lda + c];
        if (vec) v += bf2f(vec[c]);
        xr[c] = v;
    }
}

// y (+)= x / sqrt(mean(x^2) + eps) * (w_off + w[c])
__global__ void __launch_bounds__(256) k_rmsnorm_offset(const float *__restrict__ x, size_t ldx, int cols, const bf16_t *__restrict__ w, float w_off, float eps,
                                                        int accumulate, float *__restrict__ y, size_t ldy)
{
    __shared__ float red[17];
    const float *xr = x + (size_t)blockIdx.x * ldx;
    float *yr = y + (size_t)blockIdx.x * ldy;
    float q = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) q = fmaf(xr[c], xr[c], q);
    const float rinv = 1.0f / sqrtf(block_sum(q, red) / (float)cols + eps);
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = xr[c] * rinv * (w_off + (w ? bf2f(w[c]) : 0.0f));
        yr[c] = accumulate ? yr[c] + v : v;
    }
}

// What lies between two sub-layers of a block with norms on both sides of each, one workgroup per row:
//   x += m / sqrt(mean(m^2) + eps) * (w_off + w_after[c]);   h = x / sqrt(mean(x^2) + eps) * (w_off + w_before[c])   (w_before null: no h)
// The thread that updates x[c] is the one that reads it again for h.
__global__ void __launch_bounds__(256) k_norm_add_norm(float *__restrict__ x, size_t ldx, int cols, const float *__restrict__ m, size_t ldm,
                                                       const bf16_t *__restrict__ w_after, const bf16_t *__restrict__ w_before, float w_off, float eps,
                                                       float *__restrict__ h, size_t ldh)
{
    __shared__ float red[17];
    float *xr = x + (size_t)blockIdx.x * ldx;
    const float *mr = m + (size_t)blockIdx.x * ldm;
    float q = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) q = fmaf(mr[c], mr[c], q);
    const float rinv = 1.0f / sqrtf(block_sum(q, red) / (float)cols + eps);
    float q2 = 0.0f;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) {
        const float v = xr[c] + mr[c] * rinv * (w_off + bf2f(w_after[c]));
        xr[c] = v;
        q2 = fmaf(v, v, q2);
    }
    if (!w_before) return;
    const float rinv2 = 1.0f / sqrtf(block_sum(q2, red) / (float)cols + eps);
    float *hr = h + (size_t)blockIdx.x * ldh;
    for (int c = threadIdx.x; c < cols; c += blockDim.x) hr[c] = xr[c] * rinv2 * (w_off + bf2f(w_before[c]));
}

// stack[count - 1] <- x; x <- sum_j w[j] stack[j]  (element-wise over n = rows * cols values)
__global__ void __launch_bounds__(256) k_depth_average(float *__restrict__ x, size_t n, float *__restrict__ stack, size_t plane, int count, const bf16_t *__restrict__ w)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float cur = x[i];
    stack[(size_t)(count - 1) * plane + i] = cur;
    float s = 0.0f;
    for (int j = 0; j + 1 < count; j++) s = fmaf(bf2f(w[j]), stack[(size_t)j * plane + i], s);
    x[i] = fmaf(bf2f(w[count - 1]), cur, s);
}

__global__ void __launch_bounds__(256) k_softcap(float *__restrict__ x, size_t n, float cap)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = cap * tanhf(x[i] / cap);
}

// out[t][c] = act(gu[t][c]) * gu[t][F + c]  [* sigmoid(row_gate[t])];  kind 3: the clamped form g sigmoid(1.702 g) (u + 1)
__global__ void __launch_bounds__(256) k_glu_f32(int kind, float limit, const float *__restrict__ gu, size_t ld, int F, const float *__restrict__ row_gate, size_t ldg,
                                                 float *__restrict__ out, size_t ldo)
{
    const float *g = gu + (size_t)blockIdx.y * ld;
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= F) return;
    const float a = g[c], u = g[F + c];
    float r;
    if (kind == 3) {
        const float gc = fminf(a, limit), uc = fminf(fmaxf(u, -limit), limit);
        r = gc * sigmoid_f(1.702f * gc) * (uc + 1.0f);
    } else {
        const float act = kind == 0 ? silu_exact(a) : (kind == 1 ? gelu_tanh_f(a) : fmaxf(a, 0.0f));
        r = act * u;
    }
    if (row_gate) r *= sigmoid_f(row_gate[(size_t)blockIdx.y * ldg]);
    out[(size_t)blockIdx.y * ldo + c] = r;
}

__global__ void __launch_bounds__(1024) k_argmax_f32(const float *__restrict__ logits, int n, size_t row_stride, const int *__restrict__ excluded,
                                                    int *__restrict__ out)
{
    __shared__ float bv[16]; __shared__ int bi[16];
    const float *r = logits + (size_t)blockIdx.x * row_stride;
    int ex[3] = {-1, -1, -1};
    if (excluded) { const int ne = min(excluded[0], 3); for (int e = 0; e < ne; e++) ex[e] = excluded[1 + e]; }
    float best = -INFINITY; int idx = 0x7FFFFFFF;
    for (int c = threadIdx.x; c < n; c += blockDim.x) {
        if (c == ex[0] || c == ex[1] || c == ex[2]) continue;
        const float v = r[c];
        if (v > best || (v == best && c < idx)) { best = v; idx = c; }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(best, o, 64); const int oi = __shfl_xor(idx, o, 64);
        if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
    }
    if ((threadIdx.x & 63) == 0) { bv[threadIdx.x >> 6] = best; bi[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < (int)(blockDim.x >> 6); w++) if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
        out[blockIdx.x] = idx == 0x7FFFFFFF ? 0 : idx;
    }
}

__global__ void __launch_bounds__(256) k_f32_to_f16(const float *__restrict__ src, size_t n, _Float16 *__restrict__ dst)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = (_Float16)src[i];
}

} // namespace

extern "C" {

int ifa_embed_sinpos_f32(const void *embed_bf16, int vocab, int width, const int *tokens_dev, const int *positions_dev, size_t tokens,
                         float base, void *x_f32, ifa_stream stream)
{
    IFA_REQUIRE(embed_bf16 && tokens_dev && positions_dev && x_f32, "ifa_embed_sinpos_f32: null pointer");
    IFA_REQUIRE(vocab > 0 && width > 0 && tokens > 0 && base > 1.0f, "ifa_embed_sinpos_f32: bad shape");
    hipLaunchKernelGGL(k_embed_sinpos, dim3((unsigned)tokens), dim3(256), 0, ifa_s(stream), (const bf16_t *)embed_bf16, vocab, width, tokens_dev,
                       positions_dev, log((double)base), (float *)x_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_embed_rows_f32(const void *embed_bf16, int vocab, int width, const int *tokens_dev, size_t tokens, void *x_f32, ifa_stream stream)
{
    IFA_REQUIRE(embed_bf16 && tokens_dev && x_f32, "ifa_embed_rows_f32: null pointer");
    IFA_REQUIRE(vocab > 0 && width > 0 && tokens > 0, "ifa_embed_rows_f32: bad shape");
    hipLaunchKernelGGL(k_embed_rows, dim3((unsigned)tokens), dim3(256), 0, ifa_s(stream), (const bf16_t *)embed_bf16, vocab, width, tokens_dev, (float *)x_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_group_rmsnorm_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, int groups, const void *w_bf16, float eps, int accumulate,
                          void *y_f32, size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && y_f32, "ifa_group_rmsnorm_f32: null pointer");
    IFA_REQUIRE(rows > 0 && cols > 0 && groups >= 1 && cols % (size_t)groups == 0 && ldx >= cols && ldy >= cols, "ifa_group_rmsnorm_f32: bad arguments (%zu columns in %d parts)", cols, groups);
    IFA_REQUIRE(!accumulate || x_f32 != y_f32, "ifa_group_rmsnorm_f32: accumulating a row's norm into the row itself");
    hipLaunchKernelGGL(k_group_rmsnorm, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const float *)x_f32, ldx, (int)cols, groups, (const bf16_t *)w_bf16, eps,
                       accumulate ? 1 : 0, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_depth_average_f32(void *x_f32, size_t rows, size_t cols, void *stack_f32, size_t plane_stride, int count, const void *w_bf16, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && stack_f32 && w_bf16, "ifa_depth_average_f32: null pointer");
    IFA_REQUIRE(rows > 0 && cols > 0 && count >= 1 && plane_stride >= rows * cols, "ifa_depth_average_f32: bad arguments");
    const size_t n = rows * cols;
    hipLaunchKernelGGL(k_depth_average, dim3(ifa_cdiv(n, 256)), dim3(256), 0, ifa_s(stream), (float *)x_f32, n, (float *)stack_f32, plane_stride, count, (const bf16_t *)w_bf16);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_softcap_f32(void *x_f32, size_t n, float cap, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && n > 0 && cap > 0.0f, "ifa_softcap_f32: bad arguments");
    hipLaunchKernelGGL(k_softcap, dim3(ifa_cdiv(n, 256)), dim3(256), 0, ifa_s(stream), (float *)x_f32, n, cap);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_layernorm_f32(int kind, const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *w_bf16, float eps, void *y_f32, size_t ldy,
                      ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && y_f32, "ifa_layernorm_f32: null pointer");
    IFA_REQUIRE((kind == 0 || kind == 1) && rows > 0 && cols > 0 && ldx >= cols && ldy >= cols, "ifa_layernorm_f32: bad arguments");
    hipLaunchKernelGGL(k_norm_f32, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), kind, (const float *)x_f32, ldx, (int)cols,
                       (const bf16_t *)w_bf16, eps, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_glu_f32(int kind, const void *gate_up_f32, size_t ld, size_t rows, size_t cols, void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(gate_up_f32 && out_f32, "ifa_glu_f32: null pointer");
    IFA_REQUIRE(kind >= 0 && kind <= 2 && rows > 0 && cols > 0 && ld >= 2 * cols && ldo >= cols, "ifa_glu_f32: bad arguments");
    hipLaunchKernelGGL(k_glu_f32, dim3(ifa_cdiv(cols, 256), (unsigned)rows), dim3(256), 0, ifa_s(stream), kind, 0.0f, (const float *)gate_up_f32, ld,
                       (int)cols, (const float *)nullptr, (size_t)0, (float *)out_f32, ldo);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_glu_ex_f32(int kind, float limit, const void *gate_up_f32, size_t ld, size_t rows, size_t cols, const void *row_gate_f32, size_t ldg,
                   void *out_f32, size_t ldo, ifa_stream stream)
{
    IFA_REQUIRE(gate_up_f32 && out_f32, "ifa_glu_ex_f32: null pointer");
    IFA_REQUIRE(kind >= 0 && kind <= 3 && rows > 0 && cols > 0 && ld >= 2 * cols && ldo >= cols && (kind != 3 || limit > 0.0f), "ifa_glu_ex_f32: bad arguments");
    hipLaunchKernelGGL(k_glu_f32, dim3(ifa_cdiv(cols, 256), (unsigned)rows), dim3(256), 0, ifa_s(stream), kind, limit, (const float *)gate_up_f32, ld,
                       (int)cols, (const float *)row_gate_f32, ldg, (float *)out_f32, ldo);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_embed_pair_f32(const void *embed_bf16, int vocab, int width, const void *pair_bf16, int buckets, int mul_prev, int mul_cur, const int *tokens_dev,
                       const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t state_off, void *x_f32,
                       ifa_stream stream)
{
    IFA_REQUIRE(embed_bf16 && tokens_dev && seqs_dev && row_seq_dev && slot_base_dev && x_f32, "ifa_embed_pair_f32: null pointer");
    IFA_REQUIRE(vocab > 0 && width > 0 && rows > 0 && (!pair_bf16 || buckets > 0), "ifa_embed_pair_f32: bad shape");
    hipLaunchKernelGGL(k_embed_pair, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const bf16_t *)embed_bf16, vocab, width, (const bf16_t *)pair_bf16, buckets,
                       mul_prev, mul_cur, tokens_dev, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, state_off, (float *)x_f32, 1.0f,
                       (float *)nullptr);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_embed_pair_scaled_f32(const void *embed_bf16, int vocab, int width, float embed_scale, const void *pair_bf16, int buckets, int mul_prev, int mul_cur,
                              const int *tokens_dev, const void *seqs_dev, const int *row_seq_dev, size_t rows, void *const *slot_base_dev, size_t state_off,
                              void *x_f32, void *x_copy_f32, ifa_stream stream)
{
    IFA_REQUIRE(embed_bf16 && tokens_dev && seqs_dev && row_seq_dev && slot_base_dev && x_f32, "ifa_embed_pair_scaled_f32: null pointer");
    IFA_REQUIRE(vocab > 0 && width > 0 && rows > 0 && (!pair_bf16 || buckets > 0), "ifa_embed_pair_scaled_f32: bad shape");
    hipLaunchKernelGGL(k_embed_pair, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const bf16_t *)embed_bf16, vocab, width, (const bf16_t *)pair_bf16, buckets,
                       mul_prev, mul_cur, tokens_dev, (const SeqDesc *)seqs_dev, row_seq_dev, (float *const *)slot_base_dev, state_off, (float *)x_f32, embed_scale,
                       (float *)x_copy_f32);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

static dim3 rows_grid(size_t rows, size_t cols) { return dim3((unsigned)rows, (unsigned)std::min<size_t>(16, (cols + 255) / 256)); }

int ifa_dyt_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *alpha_bf16, const void *w_bf16, const void *b_bf16, void *y_f32,
                size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && alpha_bf16 && w_bf16 && b_bf16 && y_f32, "ifa_dyt_f32: null pointer");
    IFA_REQUIRE(rows > 0 && rows < (1u << 31) && cols > 0 && ldx >= cols && ldy >= cols, "ifa_dyt_f32: bad arguments");
    hipLaunchKernelGGL(k_dyt, rows_grid(rows, cols), dim3(256), 0, ifa_s(stream), (const float *)x_f32, ldx, (int)cols, (const bf16_t *)alpha_bf16,
                       (const bf16_t *)w_bf16, (const bf16_t *)b_bf16, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_add_dyt_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *vec_bf16, const void *alpha_bf16, const void *w_bf16,
                    const void *b_bf16, void *h_f32, size_t ldh, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && (!w_bf16 || (alpha_bf16 && b_bf16 && h_f32)), "ifa_add_dyt_f32: null pointer");
    IFA_REQUIRE(rows > 0 && rows < (1u << 31) && cols > 0 && ldx >= cols && (!m_f32 || ldm >= cols) && (!w_bf16 || ldh >= cols), "ifa_add_dyt_f32: bad arguments");
    if (!m_f32 && !vec_bf16 && !w_bf16) return IFA_OK;
    hipLaunchKernelGGL(k_add_dyt, rows_grid(rows, cols), dim3(256), 0, ifa_s(stream), (float *)x_f32, ldx, (int)cols, (const float *)m_f32, ldm, (const bf16_t *)vec_bf16,
                       (const bf16_t *)alpha_bf16, (const bf16_t *)w_bf16, (const bf16_t *)b_bf16, (float *)h_f32, ldh);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_add_rows_vec_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *add_f32, size_t lda, const void *vec_bf16, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && rows > 0 && rows < (1u << 31) && cols > 0 && ldx >= cols && (!add_f32 || lda >= cols), "ifa_add_rows_vec_f32: bad arguments");
    if (!add_f32 && !vec_bf16) return IFA_OK;
    hipLaunchKernelGGL(k_add_rows_vec, rows_grid(rows, cols), dim3(256), 0, ifa_s(stream), (float *)x_f32, ldx, (int)cols, (const float *)add_f32, lda,
                       (const bf16_t *)vec_bf16);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_rmsnorm_offset_f32(const void *x_f32, size_t ldx, size_t rows, size_t cols, const void *w_bf16, float w_offset, float eps, int accumulate,
                           void *y_f32, size_t ldy, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && y_f32, "ifa_rmsnorm_offset_f32: null pointer");
    IFA_REQUIRE(rows > 0 && cols > 0 && ldx >= cols && ldy >= cols, "ifa_rmsnorm_offset_f32: bad arguments");
    IFA_REQUIRE(!accumulate || x_f32 != y_f32, "ifa_rmsnorm_offset_f32: accumulating a row's norm into the row itself");
    hipLaunchKernelGGL(k_rmsnorm_offset, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (const float *)x_f32, ldx, (int)cols, (const bf16_t *)w_bf16, w_offset, eps,
                       accumulate ? 1 : 0, (float *)y_f32, ldy);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_argmax_rows_f32(const void *logits_f32, size_t n, size_t row_stride, size_t rows, const int *excluded_dev, int *out_dev, ifa_stream stream)
{
    IFA_REQUIRE(logits_f32 && out_dev && n > 0 && rows > 0 && n < (1u << 30), "ifa_argmax_rows_f32: bad arguments");
    hipLaunchKernelGGL(k_argmax_f32, dim3((unsigned)rows), dim3(n >= 4096 ? 1024 : 256), 0, ifa_s(stream), (const float *)logits_f32, (int)n, row_stride, excluded_dev, out_dev);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_convert_f32_f16(const void *src_f32, size_t n, void *dst_f16, ifa_stream stream)
{
    IFA_REQUIRE(src_f32 && dst_f16 && n > 0, "ifa_convert_f32_f16: bad arguments");
    hipLaunchKernelGGL(k_f32_to_f16, dim3(ifa_cdiv(n, 256)), dim3(256), 0, ifa_s(stream), (const float *)src_f32, n, (_Float16 *)dst_f16);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

int ifa_norm_add_norm_f32(void *x_f32, size_t ldx, size_t rows, size_t cols, const void *m_f32, size_t ldm, const void *w_after_bf16,
                          const void *w_before_bf16, float w_offset, float eps, void *h_f32, size_t ldh, ifa_stream stream)
{
    IFA_REQUIRE(x_f32 && m_f32 && w_after_bf16 && (!w_before_bf16 || h_f32), "ifa_norm_add_norm_f32: null pointer");
    IFA_REQUIRE(rows > 0 && cols > 0 && ldx >= cols && ldm >= cols && (!w_before_bf16 || ldh >= cols) && x_f32 != m_f32, "ifa_norm_add_norm_f32: bad arguments");
    hipLaunchKernelGGL(k_norm_add_norm, dim3((unsigned)rows), dim3(256), 0, ifa_s(stream), (float *)x_f32, ldx, (int)cols, (const float *)m_f32, ldm,
                       (const bf16_t *)w_after_bf16, (const bf16_t *)w_before_bf16, w_offset, eps, (float *)h_f32, ldh);
    IFA_LAUNCH_CHECK();
    return IFA_OK;
}

} // extern "C"
