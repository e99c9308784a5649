// Grouped-query attention over a paged key/value cache for packed steps, with the score shaping some decoder families use:
//   s_j = (q . k_j) * scale * temp[h];  s_j <- cap * tanh(s_j / cap) (cap > 0);  p = softmax over the visible j;  o = sum_j p_j v_j
// Position i of a sequence sees j <= i when i - j < window (window 0: every earlier key) or j < keep_first (the first tokens of
// the sequence stay visible after the window has passed them).  No rotation: positions only decide visibility.  Query head h
// reads key/value head h / (heads / kv_heads); key and value widths may differ.  The head's output may be multiplied by
// sigmoid(gate[t, h]) (one number per token and head, or one per output element) before it is stored.
// Extras (vmx_window_attention_ex), each optional: a learned sink per head in the softmax denominator (exp(sink), no key, no value);
// a logarithmic distance penalty s_j -= r1[h] * ln(1 + r2[h] * (i - j)) after the soft cap; mixing of the heads' scores,
// s_h <- sum_g talk[h, g] s_g at every visible key, before the softmax (all heads of a token then run in one workgroup).
// vmx_qk_prepare_cache_write readies a step's projected rows: whole-row RMS norms of q and k, pair rotation, cache write;
// vmx_qk_prepare_ex does the same head by head (norms over each head with gains shared by the heads, rotation of neighbouring
// coordinates or of the two halves of the rotated run, scaled cos / sin, constant multipliers, keys to plain rows for a mixer
// that keeps no cache).
//
// Keys and values live in two caches of rows [kv_heads * dim] / [kv_heads * vdim], bf16 or f32; a step writes its new rows first
// (vmx_kv_cache_write_f32) and prompts, prompt portions and decode tokens then run the SAME kernel over the cache, so a row's
// result does not depend on how its prompt was cut or on what else is in the step.  Scores, softmax and the weighted sum are f32.
// The visible keys of a row are two runs, [0, min(keep_first, lo)) and [lo, i] with lo = max(0, i - window + 1).  Two kernels:
// the vector form (any sizes, f32 or bf16 cache: a wave owns one (token, head) row and walks its keys 64 at a time, lane l scores
// key l of the tile, then every lane sums its value columns) and the matrix-core form below for bf16 caches.
#include "vmx_kernels.h"
#include <float.h>
#include <algorithm>

namespace {

template <bool F32> __device__ __forceinline__ float ld_cache(const void *c, int64_t i) {
    if constexpr (F32) return ((const float *)c)[i];
    else return vmx_bf16_to_f32(((const uint16_t *)c)[i]);
}

// k / v rows of the step's tokens -> cache rows slots[t] (negative: not stored)
__global__ __launch_bounds__(256) void kv_cache_write_kernel(const float *__restrict__ k, int64_t ldk, const float *__restrict__ v, int64_t ldv,
                                                              const int32_t *__restrict__ slots, void *__restrict__ kc, void *__restrict__ vc,
                                                              int f32, int kw, int vw) {
    const int t = blockIdx.x;
    const int64_t slot = slots[t];
    if (slot < 0) return;
    for (int i = threadIdx.x; i < kw + vw; i += 256) {
        const bool isk = i < kw;
        const int c = isk ? i : i - kw;
        const float x = isk ? k[(int64_t)t * ldk + c] : v[(int64_t)t * ldv + c];
        void *dst = isk ? kc : vc;
        const int64_t o = slot * (isk ? kw : vw) + c;
        if (f32) ((float *)dst)[o] = x;
        else ((uint16_t *)dst)[o] = vmx_f32_to_bf16(x);
    }
}

// tanh through one exponential, for the bf16 matrix-core form: absolute error about 1e-7, far below the bf16 rounding of its operands
__device__ __forceinline__ float tanh_fast(float y) { return 1.0f - 2.0f * __frcp_rn(1.0f + __expf(2.0f * y)); }

struct WinAttn {
    void *out;
    int out_f32;
    const float *q;
    int64_t ldq;
    const void *kc, *vc;
    const int32_t *block_tables, *seq_ids, *positions;
    int max_blocks;
    const uint16_t *temp;
    const float *gate;
    int64_t ldgate;
    float scale, softcap;
    int window, keep_first, tokens, heads, kv_heads, dim, vdim, block_size;
    const int32_t *seq_starts;   // matrix-core form: sequence s owns the packed rows seq_starts[s] .. seq_starts[s + 1] - 1
    int num_seqs;
    int bs_shift;                // log2(block_size) when it is a power of two, else -1
    int parts;                   // > 1: the key tiles of a run are dealt to `parts` workgroups, whose results go to `ws` for the merge
    float *ws;                   // [tokens, heads, parts, vdim + 2]: unnormalised sums, running maximum, denominator
    const uint16_t *sink, *r1, *r2, *talk;   // extras, each NULL when absent
    int gate_elem;               // 1: gate rows hold heads * vdim numbers
};

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// the denominator's sink term: (m, den, f) -> the running maximum with the sink in it, the denominator plus exp(sink - maximum),
// and the factor the sums gathered under the old maximum take
__device__ __forceinline__ void add_sink(float sink, float &m, float &den, float &f) {
    const float mn = fmaxf(m, sink);
    f = expf(m - mn);
    den = den * f + expf(sink - mn);
    m = mn;
}

// q_out[t] / key row of token t: optional whole-row RMS norm, optional pair rotation inside every head, keys and values to the cache
__global__ __launch_bounds__(256) void qk_prepare_kernel(float *__restrict__ q_out, const float *__restrict__ q, int64_t ldq, int qw,
                                                          const float *__restrict__ k, int64_t ldk, int kw, const float *__restrict__ v,
                                                          int64_t ldv, int vw, const uint16_t *__restrict__ qn, const uint16_t *__restrict__ kn,
                                                          float eps, const float *__restrict__ inv_freq, int rot_dims, int head_dim,
                                                          const int32_t *__restrict__ positions, const int32_t *__restrict__ slots,
                                                          void *__restrict__ kc, void *__restrict__ vc, int f32) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *qr = q + (int64_t)t * ldq, *kr = k + (int64_t)t * ldk, *vr = v + (int64_t)t * ldv;
    float qinv = 1.0f, kinv = 1.0f;
    if (qn) {
        float ss = 0.f;
        for (int i = tid; i < qw; i += 256) ss += qr[i] * qr[i];
        ss = vmx_block_sum_256(ss, red);
        qinv = 1.0f / sqrtf(ss / (float)qw + eps);
        __syncthreads();
    }
    if (kn) {
        float ss = 0.f;
        for (int i = tid; i < kw; i += 256) ss += kr[i] * kr[i];
        ss = vmx_block_sum_256(ss, red);
        kinv = 1.0f / sqrtf(ss / (float)kw + eps);
    }
    const float pos = (float)positions[t];
    const int64_t slot = slots[t];
    const bool rot = inv_freq && rot_dims > 0;
    for (int i = tid; i < qw + kw; i += 256) {
        const bool isq = i < qw;
        const int e = isq ? i : i - qw;
        const float *src = isq ? qr : kr;
        const uint16_t *w = isq ? qn : kn;
        const float inv = isq ? qinv : kinv;
        float x = src[e] * inv;
        if (w) x *= vmx_bf16_to_f32(w[e]);
        const int c = e % head_dim;
        if (rot && c < rot_dims) {
            float y = src[e ^ 1] * inv;   // the pair's other coordinate (rot_dims and head_dim are even)
            if (w) y *= vmx_bf16_to_f32(w[e ^ 1]);
            float sn, cs;
            sincosf(pos * inv_freq[c >> 1], &sn, &cs);
            x = (c & 1) ? x * cs + y * sn : x * cs - y * sn;
        }
        if (isq) q_out[(int64_t)t * qw + e] = x;
        else if (slot >= 0) {
            if (f32) ((float *)kc)[slot * kw + e] = x;
            else ((uint16_t *)kc)[slot * kw + e] = vmx_f32_to_bf16(x);
        }
    }
    if (slot >= 0)
        for (int i = tid; i < vw; i += 256) {
            if (f32) ((float *)vc)[slot * vw + i] = vr[i];
            else ((uint16_t *)vc)[slot * vw + i] = vmx_f32_to_bf16(vr[i]);
        }
}

struct QkPrep {
    float *q_out;
    const float *q, *k, *v;
    int64_t ldq, ldk, ldv;
    int qw, kw, vw;
    const uint16_t *qn, *kn;
    float eps;
    const float *inv_freq;
    int rot_dims, head_dim;
    const int32_t *positions, *slots;
    void *kc, *vc;
    int f32, rot_halves;
    float rot_mul, q_mul, k_mul;
    float *k_out;
    int64_t ldk_out;
};

// One wave per (token, query or key head): optional RMS norm over the head (gains of head_dim numbers, the same for every head),
// optional rotation of the head's first rot_dims coordinates, a constant multiplier; queries to q_out, keys to the cache row
// slots[t] or to k_out[t].  The rotation pairs coordinate i with i + rot_dims / 2 (rot_halves) or 2i with 2i + 1; the partner's
// value is recomputed from the input row, so lanes exchange nothing but the sum of squares.  Workgroups with blockIdx.y == 0 also
// store the token's value row.
__global__ __launch_bounds__(256) void qk_prepare_heads_kernel(const QkPrep a) {
    const int t = blockIdx.x, lane = threadIdx.x & 63;
    const int hh = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int qh = a.qw / a.head_dim, kh = a.kw / a.head_dim, hd = a.head_dim;
    const int64_t slot = a.slots ? a.slots[t] : -1;
    if (hh < qh + kh) {
        const bool isq = hh < qh;
        const int h = isq ? hh : hh - qh;
        const float *src = (isq ? a.q + (int64_t)t * a.ldq : a.k + (int64_t)t * a.ldk) + (int64_t)h * hd;
        const uint16_t *w = isq ? a.qn : a.kn;
        float inv = 1.0f;
        if (w) {
            float ss = 0.f;
            for (int c = lane; c < hd; c += 64) ss = fmaf(src[c], src[c], ss);
            inv = 1.0f / sqrtf(vmx_wave_sum(ss) / (float)hd + a.eps);
        }
        const float pos = (float)a.positions[t], mul = isq ? a.q_mul : a.k_mul;
        const bool rot = a.inv_freq && a.rot_dims > 0;
        const int half = a.rot_dims >> 1;
        for (int c = lane; c < hd; c += 64) {
            float x = src[c] * inv;
            if (w) x *= vmx_bf16_to_f32(w[c]);
            if (rot && c < a.rot_dims) {
                const bool second = a.rot_halves ? c >= half : (c & 1);
                const int pc = a.rot_halves ? (second ? c - half : c + half) : (c ^ 1);
                const int fi = a.rot_halves ? (second ? c - half : c) : (c >> 1);
                float y = src[pc] * inv;
                if (w) y *= vmx_bf16_to_f32(w[pc]);
                float sn, cs;
                sincosf(pos * a.inv_freq[fi], &sn, &cs);
                sn *= a.rot_mul, cs *= a.rot_mul;
                x = second ? x * cs + y * sn : x * cs - y * sn;
            }
            x *= mul;
            const int e = h * hd + c;
            if (isq) a.q_out[(int64_t)t * a.qw + e] = x;
            else if (a.k_out) a.k_out[(int64_t)t * a.ldk_out + e] = x;
            else if (slot >= 0) {
                if (a.f32) ((float *)a.kc)[slot * a.kw + e] = x;
                else ((uint16_t *)a.kc)[slot * a.kw + e] = vmx_f32_to_bf16(x);
            }
        }
    }
    if (blockIdx.y == 0 && a.v && a.vc && slot >= 0) {
        const float *vr = a.v + (int64_t)t * a.ldv;
        for (int i = threadIdx.x; i < a.vw; i += 256) {
            if (a.f32) ((float *)a.vc)[slot * a.vw + i] = vr[i];
            else ((uint16_t *)a.vc)[slot * a.vw + i] = vmx_f32_to_bf16(vr[i]);
        }
    }
}

constexpr int WA_MAX_DIM = 256;

template <bool F32, int VPL>
__global__ __launch_bounds__(256) void window_attn_wave_kernel(const WinAttn p) {
    __shared__ float qs[4][WA_MAX_DIM];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + wave;
    if (row >= p.tokens * p.heads) return;   // whole waves leave; no barrier below
    const int t = row / p.heads, h = row % p.heads, kvh = h / (p.heads / p.kv_heads);
    const int D = p.dim, V = p.vdim;
    const int64_t kw = (int64_t)p.kv_heads * D, vw = (int64_t)p.kv_heads * V;
    const int pos = p.positions[t];
    const int32_t *bt = p.block_tables + (int64_t)p.seq_ids[t] * p.max_blocks;
    const float qmul = p.scale * (p.temp ? vmx_bf16_to_f32(p.temp[h]) : 1.0f);
    for (int i = lane; i < D; i += 64) qs[wave][i] = p.q[(int64_t)t * p.ldq + (int64_t)h * D + i] * qmul;
    __builtin_amdgcn_wave_barrier();
    const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int na = min(p.keep_first, lo), n = na + (pos - lo + 1);
    const float inv_cap = p.softcap > 0.f ? 1.0f / p.softcap : 0.f;
    float m = -FLT_MAX, den = 0.f, acc[VPL];
#pragma unroll
    for (int u = 0; u < VPL; u++) acc[u] = 0.f;
    for (int base = 0; base < n; base += 64) {
        const int idx = base + lane;
        const bool live = idx < n;
        int crow = 0;
        float s = -FLT_MAX;
        if (live) {
            const int j = idx < na ? idx : lo + (idx - na);
            crow = bt[j / p.block_size] * p.block_size + j % p.block_size;
            const int64_t kb = (int64_t)crow * kw + (int64_t)kvh * D;
            float d = 0.f;
            for (int i = 0; i < D; i++) d = fmaf(qs[wave][i], ld_cache<F32>(p.kc, kb + i), d);
            s = p.softcap > 0.f ? p.softcap * tanhf(d * inv_cap) : d;
            if (p.r1) s -= vmx_bf16_to_f32(p.r1[h]) * log1pf(vmx_bf16_to_f32(p.r2[h]) * (float)(pos - j));
        }
        const float mn = fmaxf(m, vmx_wave_max(s));
        const float pj = live ? expf(s - mn) : 0.f;
        const float f = expf(m - mn);   // m = -FLT_MAX on the first tile: exp underflows to 0 and den, acc are 0 anyway
        den = den * f + vmx_wave_sum(pj);
        m = mn;
#pragma unroll
        for (int u = 0; u < VPL; u++) acc[u] *= f;
        const int cnt = min(64, n - base);
        for (int j = 0; j < cnt; j++) {
            const float w = __shfl(pj, j, 64);
            const int64_t r = __shfl(crow, j, 64);
            const int64_t vb = r * vw + (int64_t)kvh * V;
#pragma unroll
            for (int u = 0; u < VPL; u++) {
                const int c = lane + 64 * u;
                if (c < V) acc[u] = fmaf(w, ld_cache<F32>(p.vc, vb + c), acc[u]);
            }
        }
    }
    if (p.sink) {
        float f;
        add_sink(vmx_bf16_to_f32(p.sink[h]), m, den, f);
#pragma unroll
        for (int u = 0; u < VPL; u++) acc[u] *= f;
    }
    float g = 1.0f / den;
    if (p.gate && !p.gate_elem) g *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + h]);
#pragma unroll
    for (int u = 0; u < VPL; u++) {
        const int c = lane + 64 * u;
        if (c < V) {
            const int64_t o = ((int64_t)t * p.heads + h) * V + c;
            float r = acc[u] * g;
            if (p.gate && p.gate_elem) r *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + (int64_t)h * V + c]);
            if (p.out_f32) ((float *)p.out)[o] = r;
            else ((uint16_t *)p.out)[o] = vmx_f32_to_bf16(r);
        }
    }
}

// The vector form with mixed heads: a workgroup owns ONE token and all its heads (wave w the heads w, w + NW, ...; HPW of them).
// Per tile of 64 keys every wave leaves the shaped scores of its heads in LDS, then reads all heads' scores of its lane's key and
// mixes them with its heads' rows of the mixing matrix; softmax and the weighted sum go on per head as in the form above.
constexpr int TALK_MAX_HEADS = 64, TALK_MAX_QS = 8192;
template <bool F32, int VPL, int HPW>
__global__ __launch_bounds__(512) void window_attn_talk_kernel(const WinAttn p) {
    extern __shared__ float talk_lds[];
    const int H = p.heads, D = p.dim, V = p.vdim, NW = blockDim.x >> 6;
    float *qs = talk_lds, *raw = qs + H * D, *tk = raw + H * 64;   // queries [H, D], shaped scores [H, 64], mixing matrix [H, H]
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, t = blockIdx.x;
    const int qpk = H / p.kv_heads;
    const int64_t kw = (int64_t)p.kv_heads * D, vw = (int64_t)p.kv_heads * V;
    const int pos = p.positions[t];
    const int32_t *bt = p.block_tables + (int64_t)p.seq_ids[t] * p.max_blocks;
    for (int i = threadIdx.x; i < H * D; i += blockDim.x)
        qs[i] = p.q[(int64_t)t * p.ldq + i] * p.scale * (p.temp ? vmx_bf16_to_f32(p.temp[i / D]) : 1.0f);
    for (int i = threadIdx.x; i < H * H; i += blockDim.x) tk[i] = vmx_bf16_to_f32(p.talk[i]);
    __syncthreads();
    const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int na = min(p.keep_first, lo), n = na + (pos - lo + 1);
    const float inv_cap = p.softcap > 0.f ? 1.0f / p.softcap : 0.f;
    float m[HPW], den[HPW], acc[HPW][VPL];
#pragma unroll
    for (int a = 0; a < HPW; a++) {
        m[a] = -FLT_MAX, den[a] = 0.f;
#pragma unroll
        for (int u = 0; u < VPL; u++) acc[a][u] = 0.f;
    }
    for (int base = 0; base < n; base += 64) {
        const int idx = base + lane;
        const bool live = idx < n;
        const int j = idx < na ? idx : lo + (idx - na);
        const int crow = live ? bt[j / p.block_size] * p.block_size + j % p.block_size : 0;
#pragma unroll
        for (int a = 0; a < HPW; a++) {
            const int h = wave + a * NW;
            if (h < H && live) {
                const int64_t kb = (int64_t)crow * kw + (int64_t)(h / qpk) * D;
                float d = 0.f;
                for (int i = 0; i < D; i++) d = fmaf(qs[h * D + i], ld_cache<F32>(p.kc, kb + i), d);
                float sc = p.softcap > 0.f ? p.softcap * tanhf(d * inv_cap) : d;
                if (p.r1) sc -= vmx_bf16_to_f32(p.r1[h]) * log1pf(vmx_bf16_to_f32(p.r2[h]) * (float)(pos - j));
                raw[h * 64 + lane] = sc;
            }
        }
        __syncthreads();
        const int cnt = min(64, n - base);
#pragma unroll
        for (int a = 0; a < HPW; a++) {
            const int h = wave + a * NW;
            if (h >= H) continue;   // whole waves: no barrier inside
            float sc = -FLT_MAX;
            if (live) {
                sc = 0.f;
                for (int g = 0; g < H; g++) sc = fmaf(tk[h * H + g], raw[g * 64 + lane], sc);
            }
            const float mn = fmaxf(m[a], vmx_wave_max(sc));
            const float pj = live ? expf(sc - mn) : 0.f;
            const float f = expf(m[a] - mn);
            den[a] = den[a] * f + vmx_wave_sum(pj);
            m[a] = mn;
#pragma unroll
            for (int u = 0; u < VPL; u++) acc[a][u] *= f;
            const int kvh = h / qpk;
            for (int jj = 0; jj < cnt; jj++) {
                const float w = __shfl(pj, jj, 64);
                const int64_t r = __shfl(crow, jj, 64);
                const int64_t vb = r * vw + (int64_t)kvh * V;
#pragma unroll
                for (int u = 0; u < VPL; u++) {
                    const int c = lane + 64 * u;
                    if (c < V) acc[a][u] = fmaf(w, ld_cache<F32>(p.vc, vb + c), acc[a][u]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < HPW; a++) {
        const int h = wave + a * NW;
        if (h >= H) continue;
        if (p.sink) {
            float f;
            add_sink(vmx_bf16_to_f32(p.sink[h]), m[a], den[a], f);
#pragma unroll
            for (int u = 0; u < VPL; u++) acc[a][u] *= f;
        }
        float g = 1.0f / den[a];
        if (p.gate && !p.gate_elem) g *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + h]);
#pragma unroll
        for (int u = 0; u < VPL; u++) {
            const int c = lane + 64 * u;
            if (c < V) {
                const int64_t o = ((int64_t)t * H + h) * V + c;
                float r = acc[a][u] * g;
                if (p.gate && p.gate_elem) r *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + (int64_t)h * V + c]);
                if (p.out_f32) ((float *)p.out)[o] = r;
                else ((uint16_t *)p.out)[o] = vmx_f32_to_bf16(r);
            }
        }
    }
}

// Matrix-core form over a bf16 cache (dim and vdim multiples of 8, dim <= 32 DS, vdim <= 16 VS).  A workgroup owns one key/value
// head and a run of up to 16 nt consecutive rows of ONE sequence (found from seq_starts, so decode batches and unequal prompts
// need no padding); wave w owns 16 of these rows for one of the query heads that share the key/value head (nt = 4 / heads per
// key/value head, at most 4 heads per pass, the rest on blockIdx.z).  The run's visible keys, [0, min(keep, lo)) and [lo, last
// row], are walked in tiles of 64: key rows are staged row-major in LDS (one tile ahead, through registers), value rows
// transposed, with the keys of a tile permuted so that the scores a lane holds are the k slots of its next operand:
//   S^T = K Q^T   (A = key rows from LDS, B = the wave's query fragments, kept in registers): lane (c, g) gets the scores of
//                 query c against keys 16 kt + 4 g + r;
//   O^T += V^T P^T (A = transposed value rows from LDS, B = those scores after the softmax, as a bf16 pair hi + lo so that the
//                 weights keep f32 precision): lane (c, g) accumulates value columns 16 vs + 4 g + r of query c.
// Every statistic of a query therefore lives in the four lanes (c, 0..3): the softmax needs two lane exchanges per tile.
template <int DS, int VS>
__global__ __launch_bounds__(256) void window_attn_mfma_kernel(const WinAttn p) {
    constexpr int KT = 64, LDK = 32 * DS + 8, LDV = KT + 8, KCH = DS, VCH = (VS + 1) / 2;
    __shared__ __align__(16) uint16_t Ks[KT * LDK];
    __shared__ __align__(16) uint16_t Vt[16 * VS * LDV];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fl = lane & 15, fg = lane >> 4;
    const int qpk = p.heads / p.kv_heads, hq = min(qpk, 4), nt = 4 / hq, RT = 16 * nt;
    const int share = blockIdx.x % p.parts;
    int tile = blockIdx.x / p.parts, r0 = 0, nrows = 0;
    for (int s = 0; s < p.num_seqs; s++) {
        const int a = p.seq_starts[s], len = p.seq_starts[s + 1] - a, n = (len + RT - 1) / RT;
        if (tile < n) {
            r0 = a + tile * RT;
            nrows = min(RT, len - tile * RT);
            break;
        }
        tile -= n;
    }
    if (nrows <= 0) return;   // the same for the whole workgroup
    const int kvh = blockIdx.y, sub = wave / hq, hh = blockIdx.z * 4 + wave % hq;
    const bool active = sub < nt && hh < qpk && 16 * sub < nrows;
    const int head = kvh * qpk + (hh < qpk ? hh : 0);
    const int D = p.dim, V = p.vdim;
    const int64_t kw = (int64_t)p.kv_heads * D, vw = (int64_t)p.kv_heads * V;
    const int i0 = p.positions[r0], i1 = i0 + nrows - 1;
    const int lo = p.window > 0 ? max(0, i0 - p.window + 1) : 0;
    const int na = min(p.keep_first, lo), nk = na + (i1 - lo + 1);
    const int32_t *bt = p.block_tables + (int64_t)p.seq_ids[r0] * p.max_blocks;
    const uint16_t *kc = (const uint16_t *)p.kc, *vc = (const uint16_t *)p.vc;
    const int qrow = 16 * sub + fl, qi = i0 + qrow;
    const bool qlive = active && qrow < nrows;
    uint4 qf[DS];
#pragma unroll
    for (int s = 0; s < DS; s++) {
        const int k = 32 * s + 8 * fg;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (qlive && k < D) {
            const float *src = p.q + (int64_t)(r0 + qrow) * p.ldq + (int64_t)head * D + k;
            float f[8];
#pragma unroll
            for (int e = 0; e < 8; e++) f[e] = src[e];
            v = vmx_pack16x8<false>(f);
        }
        qf[s] = v;
    }
    const float smul = p.scale * (p.temp ? vmx_bf16_to_f32(p.temp[head]) : 1.0f);
    const float inv_cap = p.softcap > 0.f ? 1.0f / p.softcap : 0.f;
    const float dr1 = p.r1 ? vmx_bf16_to_f32(p.r1[head]) : 0.f, dr2 = p.r1 ? vmx_bf16_to_f32(p.r2[head]) : 0.f;
    // this workgroup's share of the run's key tiles
    const int ntile = (nk + KT - 1) / KT, per = (ntile + p.parts - 1) / p.parts;
    const int kb0 = share * per * KT, kb1 = min(nk, (share + 1) * per * KT);
    uint4 kr[KCH], vr[VCH];
    int krow[KCH], vrow[VCH];    // cache rows of the tile to fetch next: looked up one tile earlier, so that a fetch is one trip to memory
    auto cache_row = [&](int idx) -> int {
        if (idx >= nk) return 0;
        const int j = idx < na ? idx : lo + (idx - na);
        if (p.bs_shift >= 0) return (bt[j >> p.bs_shift] << p.bs_shift) + (j & (p.block_size - 1));
        return bt[j / p.block_size] * p.block_size + j % p.block_size;
    };
    auto lookup = [&](int kb) {
#pragma unroll
        for (int c = 0; c < KCH; c++) krow[c] = cache_row(kb + (tid + 256 * c) / (4 * DS));
#pragma unroll
        for (int c = 0; c < VCH; c++) vrow[c] = cache_row(kb + (tid + 256 * c) % KT);
    };
    auto fetch = [&](int kb) {
#pragma unroll
        for (int c = 0; c < KCH; c++) {
            const int ch = tid + 256 * c, kk = ch / (4 * DS), part = ch % (4 * DS);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (kb + kk < kb1 && 8 * part < D) v = *reinterpret_cast<const uint4 *>(kc + (int64_t)krow[c] * kw + (int64_t)kvh * D + 8 * part);
            kr[c] = v;
        }
#pragma unroll
        for (int c = 0; c < VCH; c++) {
            const int ch = tid + 256 * c, kk = ch % KT, part = ch / KT;   // a wave's lanes: 64 keys, so that their LDS columns differ
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ch < KT * 2 * VS && kb + kk < kb1 && 8 * part < V) v = *reinterpret_cast<const uint4 *>(vc + (int64_t)vrow[c] * vw + (int64_t)kvh * V + 8 * part);
            vr[c] = v;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < KCH; c++) {
            const int ch = tid + 256 * c, kk = ch / (4 * DS), part = ch % (4 * DS);
            *reinterpret_cast<uint4 *>(Ks + kk * LDK + 8 * part) = kr[c];
        }
#pragma unroll
        for (int c = 0; c < VCH; c++) {
            const int ch = tid + 256 * c, kk = ch % KT, part = ch / KT;
            if (ch < KT * 2 * VS) {
                // key kk of the tile sits in k slot `col`: the order in which the score registers of a lane line up as an operand
                const int col = 32 * (kk >> 5) + 8 * ((kk & 15) >> 2) + (kk & 3) + 4 * ((kk >> 4) & 1);
                const uint32_t w[4] = {vr[c].x, vr[c].y, vr[c].z, vr[c].w};
#pragma unroll
                for (int e = 0; e < 8; e++) Vt[(8 * part + e) * LDV + col] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            }
        }
    };
    float m = -FLT_MAX, den = 0.f;
    vmx_f32x4 o[VS];
#pragma unroll
    for (int v = 0; v < VS; v++) o[v] = vmx_f32x4{0.f, 0.f, 0.f, 0.f};
    lookup(kb0);
    fetch(kb0);
    lookup(kb0 + KT);
    stash();
    __syncthreads();
    for (int kb = kb0; kb < kb1; kb += KT) {
        if (kb + KT < kb1) {
            fetch(kb + KT);
            lookup(kb + 2 * KT);
        }
        if (active) {
            float sc[4][4];
            float tmax = -FLT_MAX;
#pragma unroll
            for (int kt = 0; kt < 4; kt++) {
                vmx_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < DS; s++) {
                    const uint4 a = *reinterpret_cast<const uint4 *>(Ks + (16 * kt + fl) * LDK + 32 * s + 8 * fg);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, a), __builtin_bit_cast(vmx_bf16x8, qf[s]), acc, 0, 0, 0);
                }
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int idx = kb + 16 * kt + 4 * fg + r;
                    const int j = idx < na ? idx : lo + (idx - na);
                    const bool vis = qlive && idx < kb1 && j <= qi && (p.window == 0 || qi - j < p.window || j < p.keep_first);
                    float x = acc[r] * smul;
                    if (p.softcap > 0.f) x = p.softcap * tanh_fast(x * inv_cap);
                    if (p.r1) x -= dr1 * __logf(1.0f + dr2 * (float)max(qi - j, 0));
                    sc[kt][r] = vis ? x : -FLT_MAX;
                    tmax = fmaxf(tmax, sc[kt][r]);
                }
            }
            tmax = fmaxf(tmax, vmx_lane_xor<16>(tmax));
            tmax = fmaxf(tmax, vmx_lane_xor<32>(tmax));
            const float mn = fmaxf(m, tmax);
            const float f = __expf(m - mn);
            float psum = 0.f;
#pragma unroll
            for (int kt = 0; kt < 4; kt++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    sc[kt][r] = sc[kt][r] > -FLT_MAX ? __expf(sc[kt][r] - mn) : 0.f;
                    psum += sc[kt][r];
                }
            psum += vmx_lane_xor<16>(psum);
            psum += vmx_lane_xor<32>(psum);
            den = den * f + psum;
            m = mn;
            if (__any(f != 1.0f)) {   // the maximum of some row moved: rescale what was summed so far
#pragma unroll
                for (int v = 0; v < VS; v++)
#pragma unroll
                    for (int r = 0; r < 4; r++) o[v][r] *= f;
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                float hi[8], lw[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float pv = sc[2 * u + (e >> 2)][e & 3];
                    hi[e] = vmx_bf16_to_f32(vmx_f32_to_bf16(pv));
                    lw[e] = pv - hi[e];
                }
                const uint4 bh = vmx_pack16x8<false>(hi), bl = vmx_pack16x8<false>(lw);
#pragma unroll
                for (int v = 0; v < VS; v++) {
                    const uint4 a = *reinterpret_cast<const uint4 *>(Vt + (16 * v + fl) * LDV + 32 * u + 8 * fg);
                    o[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, a), __builtin_bit_cast(vmx_bf16x8, bh), o[v], 0, 0, 0);
                    o[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, a), __builtin_bit_cast(vmx_bf16x8, bl), o[v], 0, 0, 0);
                }
            }
        }
        __syncthreads();
        if (kb + KT < kb1) {
            stash();
            __syncthreads();
        }
    }
    if (!qlive) return;
    if (p.parts > 1) {           // this share's sums as they are; the merge kernel normalises
        float *w = p.ws + (((int64_t)(r0 + qrow) * p.heads + head) * p.parts + share) * (V + 2);
#pragma unroll
        for (int v = 0; v < VS; v++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int c = 16 * v + 4 * fg + r;
                if (c < V) w[c] = o[v][r];
            }
        if (fg == 0) w[V] = m, w[V + 1] = den;
        return;
    }
    if (p.sink) {
        float f;
        add_sink(vmx_bf16_to_f32(p.sink[head]), m, den, f);
#pragma unroll
        for (int v = 0; v < VS; v++)
#pragma unroll
            for (int r = 0; r < 4; r++) o[v][r] *= f;
    }
    float g = 1.0f / den;
    if (p.gate && !p.gate_elem) g *= sigmoid_f32(p.gate[(int64_t)(r0 + qrow) * p.ldgate + head]);
#pragma unroll
    for (int v = 0; v < VS; v++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int c = 16 * v + 4 * fg + r;
            if (c < V) {
                const int64_t at = ((int64_t)(r0 + qrow) * p.heads + head) * V + c;
                float x = o[v][r] * g;
                if (p.gate && p.gate_elem) x *= sigmoid_f32(p.gate[(int64_t)(r0 + qrow) * p.ldgate + (int64_t)head * V + c]);
                if (p.out_f32) ((float *)p.out)[at] = x;
                else ((uint16_t *)p.out)[at] = vmx_f32_to_bf16(x);
            }
        }
}

// Matrix-core form with mixed heads (bf16 cache).  A workgroup of 8 waves owns 16 consecutive rows of ONE sequence and ALL heads:
// wave w the heads w, w + 8, ... (HPW of them).  The visible keys are walked in tiles of 32; the key rows of every key/value head
// are staged row-major in LDS and the value rows transposed (keys permuted as in the form above), one tile ahead through registers.
// Per tile: (A) every wave computes S^T = K Q^T of its heads, shapes the scores (scale, soft cap, distance penalty) and leaves them
// in LDS as raw[head][query][key]; (B) it reads the scores of ALL heads at its lanes' (query, key) places, mixes them with its
// heads' rows of the mixing matrix, and goes on per head as above: mask, running softmax in the four lanes of a query,
// O^T += V^T P^T with P as a bf16 pair.  Launches of few rows deal a run's key tiles to several workgroups (merge kernel below).
constexpr int TM_KT = 32, TM_NW = 8, TM_NT = 64 * TM_NW, TM_MAXCH = 4;
__host__ __device__ constexpr int tm_ldk(int ds) { return 32 * ds + 8; }
static size_t talk_mfma_lds_bytes(int heads, int kv_heads, int ds, int vs) {
    return (size_t)kv_heads * TM_KT * tm_ldk(ds) * 2 + (size_t)kv_heads * 16 * vs * (TM_KT + 8) * 2 + (size_t)heads * 16 * (TM_KT + 4) * 4 +
           (size_t)heads * ((heads + 3) & ~3) * 4;
}

template <int DS, int VS, int HPW>
__global__ __launch_bounds__(TM_NT) void talk_attn_mfma_kernel(const WinAttn p) {
    constexpr int KT = TM_KT, NW = TM_NW, NT = TM_NT, LDK = tm_ldk(DS), LDV = KT + 8, LDR = KT + 4, MAXCH = TM_MAXCH;
    extern __shared__ __align__(16) unsigned char talk_mfma_lds[];
    const int H = p.heads, G = p.kv_heads, D = p.dim, V = p.vdim, qpk = H / G;
    uint16_t *Ks = (uint16_t *)talk_mfma_lds;             // [G][KT][LDK]
    uint16_t *Vt = Ks + G * KT * LDK;                     // [G][16 VS][LDV]
    float *raw = (float *)(Vt + G * 16 * VS * LDV);       // [H][16][LDR]
    float *tk = raw + H * 16 * LDR;                       // [H][H rounded up to 4]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fl = lane & 15, fg = lane >> 4;
    const int share = blockIdx.x % p.parts;
    int tile = blockIdx.x / p.parts, r0 = 0, nrows = 0;
    for (int s = 0; s < p.num_seqs; s++) {
        const int a = p.seq_starts[s], len = p.seq_starts[s + 1] - a, n = (len + 15) / 16;
        if (tile < n) {
            r0 = a + tile * 16;
            nrows = min(16, len - tile * 16);
            break;
        }
        tile -= n;
    }
    if (nrows <= 0) return;   // the same for the whole workgroup
    const int64_t kw = (int64_t)G * D, vw = (int64_t)G * V;
    const int i0 = p.positions[r0], i1 = i0 + nrows - 1;
    const int lo = p.window > 0 ? max(0, i0 - p.window + 1) : 0;
    const int na = min(p.keep_first, lo), nk = na + (i1 - lo + 1);
    const int32_t *bt = p.block_tables + (int64_t)p.seq_ids[r0] * p.max_blocks;
    const uint16_t *kc = (const uint16_t *)p.kc, *vc = (const uint16_t *)p.vc;
    const int qi = i0 + fl;
    const bool qlive = fl < nrows;
    uint4 qf[HPW][DS];
    float smul[HPW], dr1[HPW], dr2[HPW];
#pragma unroll
    for (int a = 0; a < HPW; a++) {
        const int h = wave + NW * a;
        const bool on = h < H;
        smul[a] = p.scale * (p.temp && on ? vmx_bf16_to_f32(p.temp[h]) : 1.0f);
        dr1[a] = p.r1 && on ? vmx_bf16_to_f32(p.r1[h]) : 0.f;
        dr2[a] = p.r1 && on ? vmx_bf16_to_f32(p.r2[h]) : 0.f;
#pragma unroll
        for (int s = 0; s < DS; s++) {
            const int k = 32 * s + 8 * fg;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (on && qlive && k < D) {
                const float *src = p.q + (int64_t)(r0 + fl) * p.ldq + (int64_t)h * D + k;
                float f[8];
#pragma unroll
                for (int e = 0; e < 8; e++) f[e] = src[e];
                v = vmx_pack16x8<false>(f);
            }
            qf[a][s] = v;
        }
    }
    const int H4 = (H + 3) & ~3;   // rows of the mixing matrix padded with zeros to whole float4s
    for (int i = tid; i < H * H4; i += NT) tk[i] = i % H4 < H ? vmx_bf16_to_f32(p.talk[(i / H4) * H + i % H4]) : 0.f;
    const float inv_cap = p.softcap > 0.f ? 1.0f / p.softcap : 0.f;
    const int ntile = (nk + KT - 1) / KT, per = (ntile + p.parts - 1) / p.parts;
    const int kb0 = share * per * KT, kb1 = min(nk, (share + 1) * per * KT);
    const int nKch = KT * G * 4 * DS, nVch = KT * G * 2 * VS;
    uint4 kr[MAXCH], vr[MAXCH];
    int krow[MAXCH], vrow[MAXCH];
    auto cache_row = [&](int idx) -> int {
        if (idx >= nk) return 0;
        const int j = idx < na ? idx : lo + (idx - na);
        if (p.bs_shift >= 0) return (bt[j >> p.bs_shift] << p.bs_shift) + (j & (p.block_size - 1));
        return bt[j / p.block_size] * p.block_size + j % p.block_size;
    };
    auto lookup = [&](int kb) {
#pragma unroll
        for (int c = 0; c < MAXCH; c++) {
            const int ch = tid + NT * c;
            krow[c] = cache_row(kb + (ch / (4 * DS)) % KT);
            vrow[c] = cache_row(kb + ch % KT);
        }
    };
    auto fetch = [&](int kb) {
#pragma unroll
        for (int c = 0; c < MAXCH; c++) {
            const int ch = tid + NT * c;
            {
                const int part = ch % (4 * DS), kk = (ch / (4 * DS)) % KT, g = ch / (4 * DS * KT);
                uint4 v = make_uint4(0, 0, 0, 0);
                if (ch < nKch && kb + kk < kb1 && 8 * part < D) v = *reinterpret_cast<const uint4 *>(kc + (int64_t)krow[c] * kw + (int64_t)g * D + 8 * part);
                kr[c] = v;
            }
            {
                const int kk = ch % KT, part = (ch / KT) % (2 * VS), g = ch / (KT * 2 * VS);
                uint4 v = make_uint4(0, 0, 0, 0);
                if (ch < nVch && kb + kk < kb1 && 8 * part < V) v = *reinterpret_cast<const uint4 *>(vc + (int64_t)vrow[c] * vw + (int64_t)g * V + 8 * part);
                vr[c] = v;
            }
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < MAXCH; c++) {
            const int ch = tid + NT * c;
            if (ch < nKch) {
                const int part = ch % (4 * DS), kk = (ch / (4 * DS)) % KT, g = ch / (4 * DS * KT);
                *reinterpret_cast<uint4 *>(Ks + (g * KT + kk) * LDK + 8 * part) = kr[c];
            }
            if (ch < nVch) {
                const int kk = ch % KT, part = (ch / KT) % (2 * VS), g = ch / (KT * 2 * VS);
                const int col = 8 * ((kk & 15) >> 2) + (kk & 3) + 4 * ((kk >> 4) & 1);   // the k slot in which the score registers meet key kk
                const uint32_t w[4] = {vr[c].x, vr[c].y, vr[c].z, vr[c].w};
#pragma unroll
                for (int e = 0; e < 8; e++) Vt[(g * 16 * VS + 8 * part + e) * LDV + col] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            }
        }
    };
    float m[HPW], den[HPW];
    vmx_f32x4 o[HPW][VS];
#pragma unroll
    for (int a = 0; a < HPW; a++) {
        m[a] = -FLT_MAX, den[a] = 0.f;
#pragma unroll
        for (int v = 0; v < VS; v++) o[a][v] = vmx_f32x4{0.f, 0.f, 0.f, 0.f};
    }
    lookup(kb0);
    fetch(kb0);
    lookup(kb0 + KT);
    stash();
    __syncthreads();
    for (int kb = kb0; kb < kb1; kb += KT) {
        if (kb + KT < kb1) {
            fetch(kb + KT);
            lookup(kb + 2 * KT);
        }
        // (A) shaped scores of this wave's heads into LDS
#pragma unroll
        for (int a = 0; a < HPW; a++) {
            const int h = wave + NW * a;
            if (h < H) {
                const int g = h / qpk;
#pragma unroll
                for (int kt = 0; kt < KT / 16; kt++) {
                    vmx_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int s = 0; s < DS; s++) {
                        const uint4 ka = *reinterpret_cast<const uint4 *>(Ks + (g * KT + 16 * kt + fl) * LDK + 32 * s + 8 * fg);
                        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, ka), __builtin_bit_cast(vmx_bf16x8, qf[a][s]), acc, 0, 0, 0);
                    }
                    float4 x4;
                    float *xs = &x4.x;
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int idx = kb + 16 * kt + 4 * fg + r;
                        const int j = idx < na ? idx : lo + (idx - na);
                        float x = acc[r] * smul[a];
                        if (p.softcap > 0.f) x = p.softcap * tanh_fast(x * inv_cap);
                        if (p.r1) x -= dr1[a] * __logf(1.0f + dr2[a] * (float)max(qi - j, 0));
                        xs[r] = x;
                    }
                    *reinterpret_cast<float4 *>(raw + (h * 16 + fl) * LDR + 16 * kt + 4 * fg) = x4;
                }
            }
        }
        __syncthreads();
        // (B) mixed scores of this wave's heads, softmax, weighted values
#pragma unroll
        for (int a = 0; a < HPW; a++) {
            const int h = wave + NW * a;
            if (h < H) {
                const int g = h / qpk;
                float sc[KT / 16][4];
                float tmax = -FLT_MAX;
#pragma unroll
                for (int kt = 0; kt < KT / 16; kt++) {
                    // four heads' scores and weights are requested together, so that their LDS trips overlap
                    float4 mix = make_float4(0.f, 0.f, 0.f, 0.f);
                    for (int g2 = 0; g2 < H; g2 += 4) {
                        const float4 t4 = *reinterpret_cast<const float4 *>(tk + h * H4 + g2);
                        float4 r4[4];
#pragma unroll
                        for (int u = 0; u < 4; u++)   // past the last head: its row again, under a zero weight
                            r4[u] = *reinterpret_cast<const float4 *>(raw + (min(g2 + u, H - 1) * 16 + fl) * LDR + 16 * kt + 4 * fg);
                        const float tw[4] = {t4.x, t4.y, t4.z, t4.w};
#pragma unroll
                        for (int u = 0; u < 4; u++)
                            mix.x = fmaf(tw[u], r4[u].x, mix.x), mix.y = fmaf(tw[u], r4[u].y, mix.y), mix.z = fmaf(tw[u], r4[u].z, mix.z),
                            mix.w = fmaf(tw[u], r4[u].w, mix.w);
                    }
                    const float mx[4] = {mix.x, mix.y, mix.z, mix.w};
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const int idx = kb + 16 * kt + 4 * fg + r;
                        const int j = idx < na ? idx : lo + (idx - na);
                        const bool vis = qlive && idx < kb1 && j <= qi && (p.window == 0 || qi - j < p.window || j < p.keep_first);
                        sc[kt][r] = vis ? mx[r] : -FLT_MAX;
                        tmax = fmaxf(tmax, sc[kt][r]);
                    }
                }
                tmax = fmaxf(tmax, vmx_lane_xor<16>(tmax));
                tmax = fmaxf(tmax, vmx_lane_xor<32>(tmax));
                const float mn = fmaxf(m[a], tmax);
                const float f = __expf(m[a] - mn);
                float psum = 0.f;
#pragma unroll
                for (int kt = 0; kt < KT / 16; kt++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        sc[kt][r] = sc[kt][r] > -FLT_MAX ? __expf(sc[kt][r] - mn) : 0.f;
                        psum += sc[kt][r];
                    }
                psum += vmx_lane_xor<16>(psum);
                psum += vmx_lane_xor<32>(psum);
                den[a] = den[a] * f + psum;
                m[a] = mn;
                if (__any(f != 1.0f)) {
#pragma unroll
                    for (int v = 0; v < VS; v++)
#pragma unroll
                        for (int r = 0; r < 4; r++) o[a][v][r] *= f;
                }
                float hi[8], lw[8];
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const float pv = sc[e >> 2][e & 3];
                    hi[e] = vmx_bf16_to_f32(vmx_f32_to_bf16(pv));
                    lw[e] = pv - hi[e];
                }
                const uint4 bh = vmx_pack16x8<false>(hi), bl = vmx_pack16x8<false>(lw);
#pragma unroll
                for (int v = 0; v < VS; v++) {
                    const uint4 va = *reinterpret_cast<const uint4 *>(Vt + (g * 16 * VS + 16 * v + fl) * LDV + 8 * fg);
                    o[a][v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, va), __builtin_bit_cast(vmx_bf16x8, bh), o[a][v], 0, 0, 0);
                    o[a][v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, va), __builtin_bit_cast(vmx_bf16x8, bl), o[a][v], 0, 0, 0);
                }
            }
        }
        __syncthreads();
        if (kb + KT < kb1) {
            stash();
            __syncthreads();
        }
    }
    if (!qlive) return;
#pragma unroll
    for (int a = 0; a < HPW; a++) {
        const int h = wave + NW * a;
        if (h >= H) continue;
        if (p.parts > 1) {
            float *w = p.ws + (((int64_t)(r0 + fl) * H + h) * p.parts + share) * (V + 2);
#pragma unroll
            for (int v = 0; v < VS; v++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int c = 16 * v + 4 * fg + r;
                    if (c < V) w[c] = o[a][v][r];
                }
            if (fg == 0) w[V] = m[a], w[V + 1] = den[a];
            continue;
        }
        if (p.sink) {
            float f;
            add_sink(vmx_bf16_to_f32(p.sink[h]), m[a], den[a], f);
#pragma unroll
            for (int v = 0; v < VS; v++)
#pragma unroll
                for (int r = 0; r < 4; r++) o[a][v][r] *= f;
        }
        float gsc = 1.0f / den[a];
        if (p.gate && !p.gate_elem) gsc *= sigmoid_f32(p.gate[(int64_t)(r0 + fl) * p.ldgate + h]);
#pragma unroll
        for (int v = 0; v < VS; v++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int c = 16 * v + 4 * fg + r;
                if (c < V) {
                    const int64_t at = ((int64_t)(r0 + fl) * H + h) * V + c;
                    float x = o[a][v][r] * gsc;
                    if (p.gate && p.gate_elem) x *= sigmoid_f32(p.gate[(int64_t)(r0 + fl) * p.ldgate + (int64_t)h * V + c]);
                    if (p.out_f32) ((float *)p.out)[at] = x;
                    else ((uint16_t *)p.out)[at] = vmx_f32_to_bf16(x);
                }
            }
    }
}

template <int DS, int VS, int HPW> int talk_mfma_launch(const WinAttn &p, dim3 grid, size_t lds, hipStream_t st) {
    static bool sized = false;
    if (!sized) {
        VMX_CHECK_HIP(hipFuncSetAttribute((const void *)talk_attn_mfma_kernel<DS, VS, HPW>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        sized = true;
    }
    hipLaunchKernelGGL((talk_attn_mfma_kernel<DS, VS, HPW>), grid, dim3(TM_NT), lds, st, p);
    return VMX_OK;
}
template <int DS, int VS> int talk_mfma_launch_h(int hpw, const WinAttn &p, dim3 grid, size_t lds, hipStream_t st) {
    if (hpw == 1) return talk_mfma_launch<DS, VS, 1>(p, grid, lds, st);
    if (hpw == 2) return talk_mfma_launch<DS, VS, 2>(p, grid, lds, st);
    return talk_mfma_launch<DS, VS, 4>(p, grid, lds, st);
}

// out[t, h] = sum_p e^(m_p - M) o_p / sum_p e^(m_p - M) den_p * sigmoid(gate): the shares of a row's keys put together.  One wave
// per row: lane p takes share p's maximum and denominator (at most 32 shares), the weights are then handed round by lane reads.
__global__ __launch_bounds__(64) void window_attn_merge_kernel(const WinAttn p) {
    const int row = blockIdx.x, t = row / p.heads, h = row % p.heads, V = p.vdim, lane = threadIdx.x;
    const float *w = p.ws + (int64_t)row * p.parts * (V + 2);
    const bool mine = lane < p.parts;
    const float mq = mine ? w[lane * (V + 2) + V] : -FLT_MAX, dq = mine ? w[lane * (V + 2) + V + 1] : 0.f;
    const float sink = p.sink ? vmx_bf16_to_f32(p.sink[h]) : -FLT_MAX;
    const float M = fmaxf(vmx_wave_max(mq), sink);
    const float eq = mine ? expf(mq - M) : 0.f;            // a share without keys: e^(-huge) = 0
    float g = 1.0f / (vmx_wave_sum(eq * dq) + (p.sink ? expf(sink - M) : 0.f));
    if (p.gate && !p.gate_elem) g *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + h]);
    for (int c0 = 0; c0 < V; c0 += 64) {
        const int c = c0 + lane, cc = min(c, V - 1);
        float acc = 0.f;
        for (int q0 = 0; q0 < p.parts; q0 += 16) {         // sixteen shares' values first: independent loads, one wait
            float x[16];
#pragma unroll
            for (int q = 0; q < 16; q++) x[q] = q0 + q < p.parts ? w[(q0 + q) * (V + 2) + cc] : 0.f;
#pragma unroll
            for (int q = 0; q < 16; q++) acc = fmaf(__shfl(eq, q0 + q, 64), x[q], acc);
        }
        if (c < V) {
            const int64_t at = (int64_t)row * V + c;
            float r = acc * g;
            if (p.gate && p.gate_elem) r *= sigmoid_f32(p.gate[(int64_t)t * p.ldgate + (int64_t)h * V + c]);
            if (p.out_f32) ((float *)p.out)[at] = r;
            else ((uint16_t *)p.out)[at] = vmx_f32_to_bf16(r);
        }
    }
}

}  // namespace

extern "C" size_t vmx_window_attention_workspace_bytes(int tokens, int heads, int vdim) {
    // enough for 32 shares of up to 256 rows: launches with more rows fill the chip without splitting their keys
    return (size_t)(tokens < 256 ? tokens : 256) * heads * 32 * (vdim + 2) * 4;
}

extern "C" int vmx_kv_cache_write_f32(const float *k, int64_t ldk, const float *v, int64_t ldv, const int32_t *slots, void *k_cache,
                                      void *v_cache, int cache_dtype, int tokens, int k_width, int v_width, void *stream) {
    VMX_REQUIRE(k && v && slots && k_cache && v_cache, "kv_cache_write: null pointer");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "kv_cache_write: the cache holds f32 or bf16");
    VMX_REQUIRE(k_width >= 1 && v_width >= 1 && ldk >= k_width && ldv >= v_width, "kv_cache_write: bad row widths");
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(kv_cache_write_kernel, dim3(tokens), dim3(256), 0, vmx_stream(stream), k, ldk, v, ldv, slots, k_cache, v_cache,
                       cache_dtype == VMX_F32, k_width, v_width);
    VMX_CHECK_LAUNCH("kv_cache_write");
    return VMX_OK;
}

extern "C" int vmx_qk_prepare_cache_write(float *q_out, const float *q, int64_t ldq, int q_width, const float *k, int64_t ldk, int k_width,
                                          const float *v, int64_t ldv, int v_width, const uint16_t *q_norm_bf16, const uint16_t *k_norm_bf16,
                                          float eps, const float *inv_freq, int rot_dims, int head_dim, const int32_t *positions,
                                          const int32_t *slots, void *k_cache, void *v_cache, int cache_dtype, int tokens, void *stream) {
    VMX_REQUIRE(q_out && q && k && v && positions && slots && k_cache && v_cache, "qk_prepare: null pointer");
    VMX_REQUIRE(q_out != q, "qk_prepare: the prepared queries need rows of their own");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "qk_prepare: the cache holds f32 or bf16");
    VMX_REQUIRE(q_width >= 1 && k_width >= 1 && v_width >= 1 && ldq >= q_width && ldk >= k_width && ldv >= v_width, "qk_prepare: bad row widths");
    VMX_REQUIRE(head_dim >= 1 && q_width % head_dim == 0 && k_width % head_dim == 0, "qk_prepare: rows are not whole heads of %d", head_dim);
    const bool rot = inv_freq && rot_dims > 0;
    VMX_REQUIRE(!rot || (rot_dims % 2 == 0 && rot_dims <= head_dim && head_dim % 2 == 0),
                "qk_prepare: %d rotated coordinates in heads of %d (pairs inside a head of even size)", rot_dims, head_dim);
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(qk_prepare_kernel, dim3(tokens), dim3(256), 0, vmx_stream(stream), q_out, q, ldq, q_width, k, ldk, k_width, v, ldv, v_width,
                       q_norm_bf16, k_norm_bf16, eps, inv_freq, rot ? rot_dims : 0, head_dim, positions, slots, k_cache, v_cache,
                       cache_dtype == VMX_F32);
    VMX_CHECK_LAUNCH("qk_prepare");
    return VMX_OK;
}

extern "C" int vmx_qk_prepare_ex(float *q_out, const float *q, int64_t ldq, int q_width, const float *k, int64_t ldk, int k_width, const float *v,
                                 int64_t ldv, int v_width, const uint16_t *q_norm_bf16, const uint16_t *k_norm_bf16, float eps,
                                 const float *inv_freq, int rot_dims, int head_dim, const int32_t *positions, const int32_t *slots,
                                 void *k_cache, void *v_cache, int cache_dtype, int tokens, const vmx_qk_prepare_opts *opts, void *stream) {
    VMX_REQUIRE(opts, "qk_prepare_ex: null options");
    const vmx_qk_prepare_opts &o = *opts;
    const bool cached = o.k_out == nullptr;
    VMX_REQUIRE(q_out && q && k && positions, "qk_prepare_ex: null pointer");
    VMX_REQUIRE(!cached || (v && slots && k_cache && v_cache), "qk_prepare_ex: a cache write needs values, slots and both caches");
    VMX_REQUIRE(cached || o.ldk_out >= k_width, "qk_prepare_ex: bad key row stride");
    VMX_REQUIRE(q_out != q && o.k_out != k, "qk_prepare_ex: the prepared rows need memory of their own");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "qk_prepare_ex: the cache holds f32 or bf16");
    VMX_REQUIRE(q_width >= 1 && k_width >= 1 && ldq >= q_width && ldk >= k_width && (!cached || (v_width >= 1 && ldv >= v_width)),
                "qk_prepare_ex: bad row widths");
    VMX_REQUIRE(head_dim >= 1 && q_width % head_dim == 0 && k_width % head_dim == 0, "qk_prepare_ex: rows are not whole heads of %d", head_dim);
    VMX_REQUIRE(o.norm_per_head || (!q_norm_bf16 && !k_norm_bf16), "qk_prepare_ex: whole-row norms are vmx_qk_prepare_cache_write's");
    const bool rot = inv_freq && rot_dims > 0;
    VMX_REQUIRE(!rot || (rot_dims % 2 == 0 && rot_dims <= head_dim && (o.rot_halves || head_dim % 2 == 0)),
                "qk_prepare_ex: %d rotated coordinates in heads of %d", rot_dims, head_dim);
    if (tokens <= 0) return VMX_OK;
    const QkPrep a{q_out, q, k, cached ? v : nullptr, ldq, ldk, ldv, q_width, k_width, v_width, q_norm_bf16, k_norm_bf16, eps, inv_freq,
                   rot ? rot_dims : 0, head_dim, positions, cached ? slots : nullptr, cached ? k_cache : nullptr, cached ? v_cache : nullptr,
                   cache_dtype == VMX_F32, o.rot_halves ? 1 : 0, o.rot_mul != 0.f ? o.rot_mul : 1.0f, o.q_mul != 0.f ? o.q_mul : 1.0f,
                   o.k_mul != 0.f ? o.k_mul : 1.0f, o.k_out, o.ldk_out};
    const int heads = (q_width + k_width) / head_dim;
    hipLaunchKernelGGL(qk_prepare_heads_kernel, dim3(tokens, (heads + 3) / 4), dim3(256), 0, vmx_stream(stream), a);
    VMX_CHECK_LAUNCH("qk_prepare_ex");
    return VMX_OK;
}

extern "C" int vmx_window_attention(void *out, int out_dtype, const float *q, int64_t ldq, const void *k_cache, const void *v_cache,
                                    int cache_dtype, const int32_t *block_tables, int max_blocks_per_seq, const int32_t *seq_ids,
                                    const int32_t *positions, const uint16_t *head_temp_bf16, const float *gate, int64_t ldgate, float scale,
                                    float softcap, int window, int keep_first, int tokens, int heads, int kv_heads, int dim, int vdim,
                                    int block_size, const int32_t *seq_starts, int num_seqs, void *workspace, size_t workspace_bytes,
                                    void *stream) {
    return vmx_window_attention_ex(out, out_dtype, q, ldq, k_cache, v_cache, cache_dtype, block_tables, max_blocks_per_seq, seq_ids, positions,
                                   head_temp_bf16, gate, ldgate, scale, softcap, window, keep_first, tokens, heads, kv_heads, dim, vdim, block_size,
                                   seq_starts, num_seqs, workspace, workspace_bytes, nullptr, stream);
}

extern "C" int vmx_window_attention_ex(void *out, int out_dtype, const float *q, int64_t ldq, const void *k_cache, const void *v_cache,
                                       int cache_dtype, const int32_t *block_tables, int max_blocks_per_seq, const int32_t *seq_ids,
                                       const int32_t *positions, const uint16_t *head_temp_bf16, const float *gate, int64_t ldgate, float scale,
                                       float softcap, int window, int keep_first, int tokens, int heads, int kv_heads, int dim, int vdim,
                                       int block_size, const int32_t *seq_starts, int num_seqs, void *workspace, size_t workspace_bytes,
                                       const vmx_window_attn_extras *extras, void *stream) {
    VMX_REQUIRE(out && q && k_cache && v_cache && block_tables && seq_ids && positions, "window_attention: null pointer");
    VMX_REQUIRE((out_dtype == VMX_F32 || out_dtype == VMX_BF16) && (cache_dtype == VMX_F32 || cache_dtype == VMX_BF16),
                "window_attention: f32 or bf16 output and cache");
    VMX_REQUIRE(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0, "window_attention: %d query heads do not share %d key/value heads evenly",
                heads, kv_heads);
    VMX_REQUIRE(dim >= 1 && dim <= WA_MAX_DIM && vdim >= 1 && vdim <= 256, "window_attention: head sizes %d / %d outside 1..256", dim, vdim);
    VMX_REQUIRE(window >= 0 && keep_first >= 0 && block_size >= 1 && max_blocks_per_seq >= 1 && softcap >= 0.f, "window_attention: bad arguments");
    const vmx_window_attn_extras none = {nullptr, nullptr, nullptr, nullptr, 0};
    const vmx_window_attn_extras &ex = extras ? *extras : none;
    VMX_REQUIRE(ldq >= (int64_t)heads * dim && (!gate || ldgate >= (ex.gate_per_element ? (int64_t)heads * vdim : heads)),
                "window_attention: bad row strides");
    VMX_REQUIRE(!ex.dist_r1_bf16 == !ex.dist_r2_bf16, "window_attention: the distance penalty needs both of its numbers per head");
    VMX_REQUIRE(!ex.talk_bf16 || (heads <= TALK_MAX_HEADS && heads * dim <= TALK_MAX_QS),
                "window_attention: mixed heads take at most %d heads and %d query numbers per token", TALK_MAX_HEADS, TALK_MAX_QS);
    if (tokens <= 0) return VMX_OK;
    WinAttn p{out, out_dtype == VMX_F32, q, ldq, k_cache, v_cache, block_tables, seq_ids, positions, max_blocks_per_seq, head_temp_bf16,
              gate, ldgate, scale, softcap, window, keep_first, tokens, heads, kv_heads, dim, vdim, block_size, seq_starts, num_seqs,
              (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1, 1, (float *)workspace,
              ex.sink_bf16, ex.dist_r1_bf16, ex.dist_r2_bf16, ex.talk_bf16, ex.gate_per_element ? 1 : 0};
    hipStream_t st = vmx_stream(stream);
    const bool f32 = cache_dtype == VMX_F32;
    if (p.talk && !f32 && seq_starts && num_seqs >= 1 && dim % 8 == 0 && vdim % 8 == 0 && dim <= 256 && vdim <= 128 && ldq % 4 == 0 &&
        ((uintptr_t)q & 15) == 0 && ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)v_cache & 15) == 0 && heads <= 4 * TM_NW) {
        // all heads of 16 rows in one workgroup, on the matrix cores, when the tiles of all key/value heads fit
        const int ds = dim <= 64 ? 2 : (dim <= 128 ? 4 : 8), vs = vdim <= 32 ? 2 : (vdim <= 64 ? 4 : 8);
        const int hpw = (heads + TM_NW - 1) / TM_NW, hp = hpw <= 2 ? hpw : 4;
        const size_t lds = talk_mfma_lds_bytes(heads, kv_heads, ds, vs);
        const bool fits = (size_t)TM_KT * kv_heads * 4 * ds <= (size_t)TM_MAXCH * TM_NT && (size_t)TM_KT * kv_heads * 2 * vs <= (size_t)TM_MAXCH * TM_NT &&
                          lds <= 160 * 1024 && hp * (ds + vs) <= 40;   // staging registers, LDS, and the registers of a wave's heads
        if (fits) {
            const int runs = tokens / 16 + num_seqs;
            if (workspace && runs < 128) {
                int parts = 256 / runs < 32 ? 256 / runs : 32;   // one workgroup holds all heads: a run has few workgroups to begin with
                if (window > 0) parts = std::min(parts, (window + keep_first + 16 + TM_KT - 1) / TM_KT);
                parts = std::min<size_t>(parts, workspace_bytes / ((size_t)tokens * heads * (vdim + 2) * 4));
                if (parts > 1) p.parts = parts;
            }
            const dim3 grid(runs * p.parts);
            int rc;
#define TM_V(A)                                                              \
    (vs == 2 ? talk_mfma_launch_h<A, 2>(hp, p, grid, lds, st) : vs == 4 ? talk_mfma_launch_h<A, 4>(hp, p, grid, lds, st) \
                                                                         : talk_mfma_launch_h<A, 8>(hp, p, grid, lds, st))
            rc = ds == 2 ? TM_V(2) : (ds == 4 ? TM_V(4) : TM_V(8));
#undef TM_V
            if (rc) return rc;
            if (p.parts > 1) hipLaunchKernelGGL(window_attn_merge_kernel, dim3(tokens * heads), dim3(64), 0, st, p);
            VMX_CHECK_LAUNCH("window_attention (mixed heads, matrix cores)");
            return VMX_OK;
        }
    }
    if (p.talk) {   // all heads of a token in one workgroup
        const int nw = heads < 8 ? heads : 8, hpw = (heads + nw - 1) / nw;
        const int vpl = vdim <= 64 ? 1 : (vdim <= 128 ? 2 : 4);
        const size_t lds = ((size_t)heads * dim + (size_t)heads * 64 + (size_t)heads * heads) * 4;
        const dim3 grid(tokens), block(64 * nw);
#define WT_LAUNCH(F, U, HP) hipLaunchKernelGGL((window_attn_talk_kernel<F, U, HP>), grid, block, lds, st, p)
#define WT_HP(F, U)                         \
    do {                                    \
        if (hpw == 1) WT_LAUNCH(F, U, 1);   \
        else if (hpw == 2) WT_LAUNCH(F, U, 2); \
        else if (hpw <= 4) WT_LAUNCH(F, U, 4); \
        else WT_LAUNCH(F, U, 8);            \
    } while (0)
        if (f32) {
            if (vpl == 1) WT_HP(true, 1);
            else if (vpl == 2) WT_HP(true, 2);
            else WT_HP(true, 4);
        } else {
            if (vpl == 1) WT_HP(false, 1);
            else if (vpl == 2) WT_HP(false, 2);
            else WT_HP(false, 4);
        }
#undef WT_HP
#undef WT_LAUNCH
        VMX_CHECK_LAUNCH("window_attention (mixed heads)");
        return VMX_OK;
    }
    if (!f32 && seq_starts && num_seqs >= 1 && dim % 8 == 0 && vdim % 8 == 0 && dim <= 256 && vdim <= 128 && ldq % 4 == 0 && ((uintptr_t)q & 15) == 0 &&
        ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)v_cache & 15) == 0) {
        const int qpk = heads / kv_heads, hq = qpk < 4 ? qpk : 4, rt = 16 * (4 / hq);
        const int runs = tokens / rt + num_seqs;                              // at most one partly filled run per sequence
        const int base = runs * kv_heads * ((qpk + 3) / 4);
        if (workspace && base < 128) {   // few workgroups: deal each run's key tiles to several
            int parts = 256 / base < 16 ? 256 / base : 16;
            if (window > 0) parts = std::min(parts, (window + keep_first + rt + 63) / 64);
            parts = std::min<size_t>(parts, workspace_bytes / ((size_t)tokens * heads * (vdim + 2) * 4));
            if (parts > 1) p.parts = parts;
        }
        const dim3 mgrid(runs * p.parts, kv_heads, (qpk + 3) / 4);
        const int ds = dim <= 64 ? 2 : (dim <= 128 ? 4 : 8), vs = vdim <= 32 ? 2 : (vdim <= 64 ? 4 : 8);
#define WM_LAUNCH(A, B) hipLaunchKernelGGL((window_attn_mfma_kernel<A, B>), mgrid, dim3(256), 0, st, p)
        if (ds == 2) {
            if (vs == 2) WM_LAUNCH(2, 2);
            else if (vs == 4) WM_LAUNCH(2, 4);
            else WM_LAUNCH(2, 8);
        } else if (ds == 4) {
            if (vs == 2) WM_LAUNCH(4, 2);
            else if (vs == 4) WM_LAUNCH(4, 4);
            else WM_LAUNCH(4, 8);
        } else {
            if (vs == 2) WM_LAUNCH(8, 2);
            else if (vs == 4) WM_LAUNCH(8, 4);
            else WM_LAUNCH(8, 8);
        }
#undef WM_LAUNCH
        if (p.parts > 1) hipLaunchKernelGGL(window_attn_merge_kernel, dim3(tokens * heads), dim3(64), 0, st, p);
        VMX_CHECK_LAUNCH("window_attention (matrix cores)");
        return VMX_OK;
    }
    const dim3 grid((tokens * heads + 3) / 4), block(256);
    const int vpl = vdim <= 64 ? 1 : (vdim <= 128 ? 2 : 4);
#define WA_LAUNCH(F, U) hipLaunchKernelGGL((window_attn_wave_kernel<F, U>), grid, block, 0, st, p)
    if (f32) {
        if (vpl == 1) WA_LAUNCH(true, 1);
        else if (vpl == 2) WA_LAUNCH(true, 2);
        else WA_LAUNCH(true, 4);
    } else {
        if (vpl == 1) WA_LAUNCH(false, 1);
        else if (vpl == 2) WA_LAUNCH(false, 2);
        else WA_LAUNCH(false, 4);
    }
#undef WA_LAUNCH
    VMX_CHECK_LAUNCH("window_attention");
    return VMX_OK;
}
