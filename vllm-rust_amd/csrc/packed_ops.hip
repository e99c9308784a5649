// Kernels that every packed-step executor needs around its mixers and linears: RMS norm of the f32 residual stream (a gain per
// column or one gain for the row), the inverse map and the weighted combine of a mixture of experts whose (token, slot) pairs were
// sorted into expert blocks, greedy ids of f32 logits rows, a fill.
#include "vmx_kernels.h"
#include <float.h>

namespace {

// out[r] = x[rows ? rows[r] : r] / sqrt(mean(x^2) + eps) * w, f32 statistics; out in f32 or bf16; w one gain per column or
// (w_scalar) a single gain for the whole row.  Rows up to 4096 wide stay
// in registers between the statistic and the scaling (one trip to memory), wider rows are read twice.
__global__ __launch_bounds__(256) void rms_norm_f32in_kernel(void *__restrict__ out, int out_f32, const float *__restrict__ x,
                                                              const int32_t *__restrict__ rows, const uint16_t *__restrict__ w, int w_scalar,
                                                              int width, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float *src = x + (int64_t)(rows ? rows[r] : r) * width;
    constexpr int PT = 16;
    float xv[PT], wv[PT];
    const bool held = width <= 256 * PT;
    float ss = 0.f;
    if (held) {
#pragma unroll
        for (int u = 0; u < PT; u++) {
            const int i = threadIdx.x + 256 * u;
            xv[u] = i < width ? src[i] : 0.f;
            wv[u] = i < width ? vmx_bf16_to_f32(w[w_scalar ? 0 : i]) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < PT; u++) ss += xv[u] * xv[u];   // same order as the strided loop below
    } else {
        for (int i = threadIdx.x; i < width; i += 256) ss += src[i] * src[i];
    }
    ss = vmx_block_sum_256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)width + eps);
    if (held) {
#pragma unroll
        for (int u = 0; u < PT; u++) {
            const int i = threadIdx.x + 256 * u;
            if (i < width) {
                const float v = xv[u] * inv * wv[u];
                if (out_f32) ((float *)out)[(int64_t)r * width + i] = v;
                else ((uint16_t *)out)[(int64_t)r * width + i] = vmx_f32_to_bf16(v);
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < width; i += 256) {
        const float v = src[i] * inv * vmx_bf16_to_f32(w[w_scalar ? 0 : i]);
        if (out_f32) ((float *)out)[(int64_t)r * width + i] = v;
        else ((uint16_t *)out)[(int64_t)r * width + i] = vmx_f32_to_bf16(v);
    }
}

// Norm after the sum, over equal consecutive groups of the row: v = acc[t] (w != NULL: every group divided by its own
// sqrt(mean(group^2) + eps), then times w); x[t] = v (f32), h[t] = v (f32 or bf16: what the next products read), acc[t] = alpha * v
// (the sum the next sublayer's result is added to).  One workgroup per row, one group after the other.
__global__ __launch_bounds__(256) void group_norm_post_kernel(float *__restrict__ acc, float *__restrict__ x, void *__restrict__ h, int h_f32,
                                                               const uint16_t *__restrict__ w, int groups, int width, float eps, float alpha) {
    __shared__ float red[4];
    const int64_t row = (int64_t)blockIdx.x * width;
    const int n = width / groups;
    for (int g = 0; g < groups; g++) {
        float inv = 1.0f;
        if (w) {
            float ss = 0.f;
            for (int i = threadIdx.x; i < n; i += 256) {
                const float v = acc[row + g * n + i];
                ss = fmaf(v, v, ss);
            }
            ss = vmx_block_sum_256(ss, red);
            inv = 1.0f / sqrtf(ss / (float)n + eps);
        }
        for (int i = threadIdx.x; i < n; i += 256) {   // a thread rewrites only what it read itself
            const int c = g * n + i;
            float v = acc[row + c] * inv;
            if (w) v *= vmx_bf16_to_f32(w[c]);
            x[row + c] = v;
            if (h_f32) ((float *)h)[row + c] = v;
            else ((uint16_t *)h)[row + c] = vmx_f32_to_bf16(v);
            acc[row + c] = alpha * v;
        }
    }
}

// out[r] = x[rows ? rows[r] : r] normed in groups as above, f32 or bf16 (the rows the output matrix reads)
__global__ __launch_bounds__(256) void group_norm_rows_kernel(void *__restrict__ out, int out_f32, const float *__restrict__ x,
                                                               const int32_t *__restrict__ rows, const uint16_t *__restrict__ w, int groups,
                                                               int width, float eps) {
    __shared__ float red[4];
    const float *src = x + (int64_t)(rows ? rows[blockIdx.x] : blockIdx.x) * width;
    const int64_t row = (int64_t)blockIdx.x * width;
    const int n = width / groups;
    for (int g = 0; g < groups; g++) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(src[g * n + i], src[g * n + i], ss);
        ss = vmx_block_sum_256(ss, red);
        const float inv = 1.0f / sqrtf(ss / (float)n + eps);
        for (int i = threadIdx.x; i < n; i += 256) {
            const int c = g * n + i;
            const float v = src[c] * inv * vmx_bf16_to_f32(w[c]);
            if (out_f32) ((float *)out)[row + c] = v;
            else ((uint16_t *)out)[row + c] = vmx_f32_to_bf16(v);
        }
    }
}

// act[r, j] = silu(s g) * (s u) * sigmoid(out_gate[r]) with g = gu[r, j], u = gu[r, up_off + j]: the gated activation of an expert
// whose INPUT was scaled by s (both products are linear in their input, so the scale is applied to their results), and a
// sigmoid gate per row on what goes into the down projection (linear too).  s = in_w[in_ids ? in_ids[r] : r] (ids outside
// [0, in_limit) are padding rows: 0); in_w NULL: 1; out_gate NULL: none.
__global__ __launch_bounds__(256) void glu_silu_scaled_kernel(void *__restrict__ act, int act_f32, const float *__restrict__ gu, int64_t ldgu,
                                                               int up_off, int ff, const float *__restrict__ in_w,
                                                               const int32_t *__restrict__ in_ids, int in_limit,
                                                               const float *__restrict__ out_gate, int64_t ldgate) {
    const int64_t r = blockIdx.x;
    const int j = blockIdx.y * 256 + threadIdx.x;
    if (j >= ff) return;
    float s = 1.0f;
    if (in_w) {
        const int id = in_ids ? in_ids[r] : (int)r;
        s = (id >= 0 && id < in_limit) ? in_w[id] : 0.f;
    }
    const float g = s * gu[r * ldgu + j], u = s * gu[r * ldgu + up_off + j];
    float v = g / (1.0f + expf(-g)) * u;
    if (out_gate) v *= 1.0f / (1.0f + expf(-out_gate[r * ldgate]));
    if (act_f32) ((float *)act)[r * ff + j] = v;
    else ((uint16_t *)act)[r * ff + j] = vmx_f32_to_bf16(v);
}

// inv[pair] = position of the pair in the expert-sorted list
__global__ __launch_bounds__(256) void moe_inverse_kernel(int32_t *__restrict__ inv, const int32_t *__restrict__ sorted,
                                                           const int32_t *__restrict__ total, int numel) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < *total) {
        const int p = sorted[i];
        if (p >= 0 && p < numel) inv[p] = i;
    }
}

// x[t] += (sum_slot w[t, slot] * y[inv[t * k + slot]] (slot order) + shared[t]) * sigmoid(gate[t])   (shared, gate optional; w NULL: 1)
__global__ __launch_bounds__(256) void moe_combine_f32_kernel(float *__restrict__ x, const float *__restrict__ y,
                                                               const int32_t *__restrict__ inv, const float *__restrict__ w, int k,
                                                               const float *__restrict__ shared, const float *__restrict__ gate,
                                                               int64_t ldgate, int width) {
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;   // tokens on x (no 65535 limit)
    if (i >= width) return;
    float acc = 0.f;
    for (int s = 0; s < k; s++) acc = fmaf(w ? w[(int64_t)t * k + s] : 1.0f, y[(int64_t)inv[(int64_t)t * k + s] * width + i], acc);
    if (shared) acc += shared[(int64_t)t * width + i];
    if (gate) acc *= 1.0f / (1.0f + expf(-gate[(int64_t)t * ldgate + i]));
    x[(int64_t)t * width + i] += acc;
}

// Greedy ids in two launches: chunk winners as keys (order-preserving value bits | inverted index, so the largest key is the
// largest value with the smallest index), then the winner of a row's keys.
__device__ __forceinline__ unsigned long long argmax_key(float v, int i) {
    uint32_t b = __float_as_uint(v);
    b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((unsigned long long)b << 32) | (uint32_t)(0x7fffffff - i);
}
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const unsigned long long o = __shfl_xor(k, off, 64);
        k = o > k ? o : k;
    }
    return k;
}
__global__ __launch_bounds__(256) void argmax_f32_partial_kernel(unsigned long long *__restrict__ keys, const float *__restrict__ logits,
                                                                  int vocab, int chunks) {
    __shared__ unsigned long long red[4];
    const int r = blockIdx.y, c = blockIdx.x;
    unsigned long long best = 0;
    for (int i = c * VMX_ARGMAX_CHUNK + threadIdx.x; i < min(vocab, (c + 1) * VMX_ARGMAX_CHUNK); i += 256) {
        const unsigned long long k = argmax_key(logits[(int64_t)r * vocab + i], i);
        best = k > best ? k : best;
    }
    best = wave_max_u64(best);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w2 = 1; w2 < 4; w2++) best = red[w2] > best ? red[w2] : best;
        keys[(int64_t)r * chunks + c] = best;
    }
}
__global__ __launch_bounds__(64) void argmax_f32_final_kernel(int32_t *__restrict__ out, const unsigned long long *__restrict__ keys, int chunks) {
    const int r = blockIdx.x;
    unsigned long long best = 0;
    for (int c = threadIdx.x; c < chunks; c += 64) best = keys[(int64_t)r * chunks + c] > best ? keys[(int64_t)r * chunks + c] : best;
    best = wave_max_u64(best);
    if (threadIdx.x == 0) out[r] = best ? 0x7fffffff - (int)(uint32_t)(best & 0xffffffffu) : 0;
}

__global__ __launch_bounds__(256) void zero_f32_kernel(float *__restrict__ p, int64_t n) {
    for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) p[i] = 0.f;
}

// x[t] = embed[token] * scale (bf16 table, f32 rows); ids outside the table are clamped
__global__ __launch_bounds__(256) void embed_scaled_f32_kernel(float *__restrict__ x, const uint16_t *__restrict__ embed,
                                                                const int32_t *__restrict__ tokens, int width, int vocab, float scale) {
    const int t = blockIdx.x;
    int id = tokens[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int i = threadIdx.x; i < width; i += 256) x[(int64_t)t * width + i] = vmx_bf16_to_f32(embed[(int64_t)id * width + i]) * scale;
}

// act[r, j] = silu(gu[r, j]) * gu[r, ff + j]: the gated activation between the two products of a feed-forward whose gate and up
// projections were computed as one product
__global__ __launch_bounds__(256) void glu_silu_kernel(void *__restrict__ act, int act_f32, const float *__restrict__ gu, int ff) {
    const int64_t r = blockIdx.x;             // rows on x: a prompt's (token, expert) pairs can pass the 65535 of the other axes
    const int j = blockIdx.y * 256 + threadIdx.x;
    if (j >= ff) return;
    const float g = gu[r * 2 * ff + j], u = gu[r * 2 * ff + ff + j];
    const float v = g / (1.0f + expf(-g)) * u;
    if (act_f32) ((float *)act)[r * ff + j] = v;
    else ((uint16_t *)act)[r * ff + j] = vmx_f32_to_bf16(v);
}

// out[t] = [a[t] | b[t]] (two f32 rows of `width` numbers side by side), in f32 or bf16: the input of a product over both
__global__ __launch_bounds__(256) void concat2_rows_kernel(void *__restrict__ out, int out_f32, const float *__restrict__ a,
                                                            const float *__restrict__ b, int width) {
    const int t = blockIdx.x, i = blockIdx.y * 256 + threadIdx.x;
    if (i >= 2 * width) return;
    const float v = i < width ? a[(int64_t)t * width + i] : b[(int64_t)t * width + i - width];
    const int64_t o = (int64_t)t * 2 * width + i;
    if (out_f32) ((float *)out)[o] = v;
    else ((uint16_t *)out)[o] = vmx_f32_to_bf16(v);
}

// x <- cap * tanh(x * scale / cap) (cap 0: x * scale)
__global__ __launch_bounds__(256) void scale_softcap_kernel(float *__restrict__ x, int64_t n, float scale, float cap) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const float v = x[i] * scale;
    x[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

}  // namespace

int vmx_embed_scaled_f32(float *x, const uint16_t *embed, const int32_t *tokens, int T, int width, int vocab, float scale, hipStream_t st) {
    hipLaunchKernelGGL(embed_scaled_f32_kernel, dim3(T), dim3(256), 0, st, x, embed, tokens, width, vocab, scale);
    VMX_CHECK_LAUNCH("embed");
    return VMX_OK;
}

int vmx_glu_silu_rows(void *act, int act_f32, const float *gu, int rows, int ff, hipStream_t st) {
    if (rows <= 0) return VMX_OK;
    hipLaunchKernelGGL(glu_silu_kernel, dim3(rows, (ff + 255) / 256), dim3(256), 0, st, act, act_f32, gu, ff);
    VMX_CHECK_LAUNCH("glu silu");
    return VMX_OK;
}

int vmx_rms_norm_f32in(void *out, int out_f32, const float *x, const int32_t *rows, const uint16_t *w, int w_scalar, int width, float eps,
                       int n, hipStream_t st) {
    if (n <= 0) return VMX_OK;
    hipLaunchKernelGGL(rms_norm_f32in_kernel, dim3(n), dim3(256), 0, st, out, out_f32, x, rows, w, w_scalar, width, eps);
    VMX_CHECK_LAUNCH("rms norm");
    return VMX_OK;
}

int vmx_group_norm_post(float *acc, float *x, void *h, int h_f32, const uint16_t *w, int groups, int width, float eps, float alpha, int n,
                        hipStream_t st) {
    VMX_REQUIRE(acc && x && h && groups >= 1 && width % groups == 0, "group norm: %d groups do not divide a row of %d", groups, width);
    if (n <= 0) return VMX_OK;
    hipLaunchKernelGGL(group_norm_post_kernel, dim3(n), dim3(256), 0, st, acc, x, h, h_f32, w, groups, width, eps, alpha);
    VMX_CHECK_LAUNCH("group norm");
    return VMX_OK;
}

int vmx_group_norm_rows(void *out, int out_f32, const float *x, const int32_t *rows, const uint16_t *w, int groups, int width, float eps, int n,
                        hipStream_t st) {
    VMX_REQUIRE(out && x && w && groups >= 1 && width % groups == 0, "group norm: %d groups do not divide a row of %d", groups, width);
    if (n <= 0) return VMX_OK;
    hipLaunchKernelGGL(group_norm_rows_kernel, dim3(n), dim3(256), 0, st, out, out_f32, x, rows, w, groups, width, eps);
    VMX_CHECK_LAUNCH("group norm rows");
    return VMX_OK;
}

int vmx_glu_silu_rows_scaled(void *act, int act_f32, const float *gu, int64_t ldgu, int up_off, int rows, int ff, const float *in_w,
                             const int32_t *in_ids, int in_limit, const float *out_gate, int64_t ldgate, hipStream_t st) {
    if (rows <= 0) return VMX_OK;
    hipLaunchKernelGGL(glu_silu_scaled_kernel, dim3(rows, (ff + 255) / 256), dim3(256), 0, st, act, act_f32, gu, ldgu, up_off, ff, in_w, in_ids,
                       in_limit, out_gate, ldgate);
    VMX_CHECK_LAUNCH("glu silu (scaled)");
    return VMX_OK;
}

int vmx_zero_f32(float *p, int64_t n, hipStream_t st) {
    hipLaunchKernelGGL(zero_f32_kernel, dim3(1024), dim3(256), 0, st, p, n);
    VMX_CHECK_LAUNCH("zero");
    return VMX_OK;
}

int vmx_moe_inverse(int32_t *inv, const int32_t *sorted, const int32_t *total, int numel, int cap, hipStream_t st) {
    hipLaunchKernelGGL(moe_inverse_kernel, dim3((cap + 255) / 256), dim3(256), 0, st, inv, sorted, total, numel);
    VMX_CHECK_LAUNCH("moe inverse");
    return VMX_OK;
}

int vmx_moe_combine_f32(float *x, const float *y, const int32_t *inv, const float *w, int k, const float *shared, const float *gate,
                        int64_t ldgate, int T, int width, hipStream_t st) {
    hipLaunchKernelGGL(moe_combine_f32_kernel, dim3(T, (width + 255) / 256), dim3(256), 0, st, x, y, inv, w, k, shared, gate, ldgate, width);
    VMX_CHECK_LAUNCH("moe combine");
    return VMX_OK;
}

int vmx_argmax_f32_rows(int32_t *out, unsigned long long *keys, const float *logits, int rows, int vocab, hipStream_t st) {
    const int chunks = (vocab + VMX_ARGMAX_CHUNK - 1) / VMX_ARGMAX_CHUNK;
    hipLaunchKernelGGL(argmax_f32_partial_kernel, dim3(chunks, rows), dim3(256), 0, st, keys, logits, vocab, chunks);
    hipLaunchKernelGGL(argmax_f32_final_kernel, dim3(rows), dim3(64), 0, st, out, keys, chunks);
    VMX_CHECK_LAUNCH("argmax");
    return VMX_OK;
}

int vmx_concat2_rows(void *out, int out_f32, const float *a, const float *b, int T, int width, hipStream_t st) {
    if (T <= 0) return VMX_OK;
    hipLaunchKernelGGL(concat2_rows_kernel, dim3(T, (2 * width + 255) / 256), dim3(256), 0, st, out, out_f32, a, b, width);
    VMX_CHECK_LAUNCH("concat rows");
    return VMX_OK;
}

int vmx_scale_softcap_f32(float *x, int64_t n, float scale, float cap, hipStream_t st) {
    if (n <= 0) return VMX_OK;
    hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, x, n, scale, cap);
    VMX_CHECK_LAUNCH("scale + soft cap");
    return VMX_OK;
}
