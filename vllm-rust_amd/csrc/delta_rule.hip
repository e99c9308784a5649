// Linear recurrences over a matrix memory per head, as recurrent token mixers over packed steps (the gated delta rule with one
// decay per key channel or per head; the plain decayed outer-product memory of gated linear attention and retention), and the
// short causal convolution in front of the delta rule.  Both carry state from step to step in a SLOT per sequence (the caller's state-slot manager hands
// them out); a sequence whose step starts at position 0 starts from zeros whatever its slot held before.
//
// Short convolution (vmx_short_conv_silu): y[t, c] = silu(sum_s taps[c, n - 1 - s] * x[t - s, c]), zeros before the sequence's
// first token.  The last n - 1 inputs of every sequence are its state [slots, n - 1, channels] (f32); inputs older than the step
// come from there.  A group of channels (one head's query or key) may then be scaled to a unit vector, x / sqrt(sum x^2 + eps),
// times a constant.  vmx_short_conv_state_update moves the state on after all of a step's rows were read.
//
// Recurrence (vmx_gated_delta_rule), per head with a matrix memory S [dim, vdim] in f32:
//   S <- diag(g_t) S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t
// so a token reads the memory after its own write (computed as (g S)^T q + u (k . q), the same sum in another order).  The decay
// g_t is a number per key channel, or one per head (per token, or a constant of the head: row stride 0); without beta the write
// is the plain outer product, u = v_t (S <- diag(g_t) S + k_t v_t^T: gated linear attention, retention).  Query/key
// head of value head h: h / (heads / qk_heads).  A workgroup owns 16 value columns of one (sequence, head) and walks the
// sequence's tokens of the step in order; 16 threads share a column, each holding every 16th row of S in registers, and the
// column sums per token are 16-lane butterflies.  The state slot keeps S in the workgroup's own register order (the layout is
// private to this kernel), so that loading and storing it is coalesced.
#include "vmx_kernels.h"

namespace {

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

struct ConvArgs {
    const float *x;          // [tokens, ldx] inputs of the step, channels at column 0
    int64_t ldx;
    const uint16_t *taps;    // bf16 [channels, n]
    float *state;            // [slots, n - 1, channels]
    float *y;                // [tokens, ldy]
    int64_t ldy;
    const int32_t *positions, *seq_ids, *seq_starts, *state_slots;
    int tokens, channels, n;
    // unit-vector groups: channels [0, unit_groups * group) are groups of `group` channels; groups < scaled_groups also get `mul`
    int group, unit_groups, scaled_groups;
    float unit_eps, mul;
};

// one wave per (token, run of `group` channels); runs past the unit groups are plain 64-channel runs
__global__ __launch_bounds__(256) void short_conv_silu_kernel(const ConvArgs a) {
    const int t = blockIdx.x, lane = threadIdx.x & 63;   // tokens on x (no 65535 limit)
    const int run = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int unit_ch = a.unit_groups * a.group;
    int c0, c1;
    bool unit = false;
    if (run < a.unit_groups) c0 = run * a.group, c1 = c0 + a.group, unit = true;
    else c0 = unit_ch + (run - a.unit_groups) * 64, c1 = min(c0 + 64, a.channels);
    if (c0 >= a.channels) return;
    const int pos = a.positions[t], seq = a.seq_ids[t];
    const int first = a.seq_starts[seq];             // packed row of the sequence's first token in this step
    const int start = pos - (t - first);             // position of that token
    const float *st = a.state + (int64_t)a.state_slots[seq] * (a.n - 1) * a.channels;
    auto conv_at = [&](int c) {
        float acc = 0.f;
        for (int s = a.n - 1; s >= 0; s--) {         // oldest input first
            const int q = pos - s;
            if (q < 0) continue;
            const float xv = q >= start ? a.x[(int64_t)(t - s) * a.ldx + c] : st[(int64_t)(q - start + a.n - 1) * a.channels + c];
            acc = fmaf(vmx_bf16_to_f32(a.taps[(int64_t)c * a.n + (a.n - 1 - s)]), xv, acc);
        }
        return silu_f(acc);
    };
    constexpr int HOLD = 4;                          // a lane's outputs of a run of up to 256 channels stay in registers
    float held[HOLD], ss = 0.f;
#pragma unroll
    for (int i = 0; i < HOLD; i++) {
        const int c = c0 + lane + 64 * i;
        held[i] = c < c1 ? conv_at(c) : 0.f;
        ss = fmaf(held[i], held[i], ss);
    }
    for (int c = c0 + lane + 64 * HOLD; c < c1; c += 64) {   // wider runs go through memory
        const float yv = conv_at(c);
        a.y[(int64_t)t * a.ldy + c] = yv;
        ss = fmaf(yv, yv, ss);
    }
    float f = 1.0f;
    if (unit) f = (run < a.scaled_groups ? a.mul : 1.0f) / sqrtf(vmx_wave_sum(ss) + a.unit_eps);
#pragma unroll
    for (int i = 0; i < HOLD; i++) {
        const int c = c0 + lane + 64 * i;
        if (c < c1) a.y[(int64_t)t * a.ldy + c] = held[i] * f;
    }
    if (unit)
        for (int c = c0 + lane + 64 * HOLD; c < c1; c += 64) a.y[(int64_t)t * a.ldy + c] *= f;   // each lane rescales what it wrote itself
}

// state[slot] <- the last n - 1 inputs of the sequence after this step.  A thread owns one (sequence, channel) and goes through
// the state rows in ascending order: row r takes the input of position end - (n - 1) + r, which is a row of the step or an OLDER
// state row r + count (not overwritten yet).
__global__ __launch_bounds__(256) void short_conv_state_kernel(const ConvArgs a, int num_seqs) {
    const int seq = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if (c >= a.channels) return;
    const int first = a.seq_starts[seq], count = a.seq_starts[seq + 1] - first;
    if (count <= 0) return;
    const int start = a.positions[first];
    float *st = a.state + (int64_t)a.state_slots[seq] * (a.n - 1) * a.channels;
    for (int r = 0; r < a.n - 1; r++) {
        const int q = start + count - (a.n - 1) + r;
        float v = 0.f;
        if (q >= start) v = a.x[(int64_t)(first + q - start) * a.ldx + c];
        else if (q >= 0) v = st[(int64_t)(r + count) * a.channels + c];
        st[(int64_t)r * a.channels + c] = v;
    }
}

// g[t, c] <- exp(-exp(A_log[c / dim]) * softplus(g[t, c] + dt_bias[c])) in place, and beta[t, h] <- sigmoid(beta[t, h]) in place
__global__ __launch_bounds__(256) void delta_gates_kernel(float *__restrict__ g, int64_t ldg, const uint16_t *__restrict__ a_log,
                                                           const uint16_t *__restrict__ dt_bias, float *__restrict__ beta, int64_t ldbeta,
                                                           int heads, int dim) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c < heads * dim) {
        const float rate = expf(vmx_bf16_to_f32(a_log[c / dim]));
        const float dt = softplus_f(g[(int64_t)t * ldg + c] + vmx_bf16_to_f32(dt_bias[c]));
        g[(int64_t)t * ldg + c] = expf(-rate * dt);
    }
    if (c < heads) beta[(int64_t)t * ldbeta + c] = sigmoid_f(beta[(int64_t)t * ldbeta + c]);
}

// g[t, c] <- sigmoid(g[t, c])^(1 / tau) in place, through the logarithm: exp(-softplus(-z) / tau)
__global__ __launch_bounds__(256) void sigmoid_root_decay_kernel(float *__restrict__ g, int64_t ldg, int n, float inv_tau) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c < n) g[(int64_t)t * ldg + c] = expf(-softplus_f(-g[(int64_t)t * ldg + c]) * inv_tau);
}

struct DeltaArgs {
    const float *q, *k, *v, *g, *beta;       // rows of the step: q, k [qk_heads * dim], v [heads * vdim], g [heads * dim], beta [heads]
    int64_t ldq, ldk, ldv, ldg, ldbeta;
    float *o;                                // [tokens, heads * vdim]
    int64_t ldo;
    float *state;                            // [slots, heads, tiles, DPT, 256]
    const int32_t *positions, *seq_starts, *state_slots;
    int heads, qk_heads, dim, vdim;
    int g_per_head;                          // g rows hold one decay per head (ldg 0: the same row for every token) instead of heads * dim
    int plain;                               // no beta: u = v
    float q_mul;                             // the queries are multiplied by this constant as they are read
};

constexpr int DR_RS = 16, DR_VT = 16;   // row splits per column, columns per workgroup

// Tokens are staged in rounds of CT through two LDS buffers: the next round is requested into registers before the current one
// is walked and stored afterwards, so one barrier per round remains and the walk never waits for memory.  q, k and g are stored
// in thread order ([row split r][u] for row r + 8 u), so a thread reads its rows as 16-byte vectors.
template <int DPT>
__global__ __launch_bounds__(256) void gated_delta_rule_kernel(const DeltaArgs a) {
    constexpr int DP = DPT * DR_RS;          // padded key dimension
    constexpr int LDP = DPT == 4 ? 4 : DPT + 4;   // floats between two row splits in LDS: the 16 splits of a read fall on different banks
    constexpr int CT = 128 / DPT;            // tokens per round: long enough for the next round's loads to land while this one is walked
    constexpr int NL = CT * DP / 256;        // q / k / g elements a thread stages per round
    constexpr int NV = (CT * DR_VT + 255) / 256;
    constexpr int ROW = DR_RS * LDP;         // floats of one token's q (k, g) in LDS
    extern __shared__ __align__(16) float delta_lds[];   // delta_lds_bytes(DPT): q | k | g [2][CT][ROW], v [2][CT][16], beta [2][CT]
    float *sq = delta_lds, *sk = sq + 2 * CT * ROW, *sg = sk + 2 * CT * ROW, *sv = sg + 2 * CT * ROW, *sb = sv + 2 * CT * DR_VT;
    const int seq = blockIdx.z, h = blockIdx.y, tile = blockIdx.x, tid = threadIdx.x;
    const int first = a.seq_starts[seq], count = a.seq_starts[seq + 1] - first;
    if (count <= 0) return;
    const int r = tid & (DR_RS - 1), cl = tid >> 4, c = tile * DR_VT + cl;
    const int qh = h / (a.heads / a.qk_heads);
    const int tiles = gridDim.x;
    float *sp = a.state + ((((int64_t)a.state_slots[seq] * a.heads + h) * tiles + tile) * DPT) * 256 + tid;
    float S[DPT];
    const bool fresh = a.positions[first] == 0;
#pragma unroll
    for (int u = 0; u < DPT; u++) S[u] = fresh ? 0.f : sp[(int64_t)u * 256];
    float rq[NL], rk[NL], rg[NL], rv[NV], rb = 0.f;
    auto request = [&](int t0) {
        const int ct = min(CT, count - t0);
#pragma unroll
        for (int j = 0; j < NL; j++) {
            const int i = tid + 256 * j, tt = i / DP, d = i % DP;
            const int64_t row = first + t0 + tt;
            const bool in = tt < ct && d < a.dim;
            rq[j] = in ? a.q[row * a.ldq + (int64_t)qh * a.dim + d] * a.q_mul : 0.f;
            rk[j] = in ? a.k[row * a.ldk + (int64_t)qh * a.dim + d] : 0.f;
            rg[j] = in ? a.g[row * a.ldg + (a.g_per_head ? (int64_t)h : (int64_t)h * a.dim + d)] : 1.f;
        }
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = tid + 256 * j, tt = i / DR_VT, cc = tile * DR_VT + i % DR_VT;
            rv[j] = (tt < ct && cc < a.vdim) ? a.v[(int64_t)(first + t0 + tt) * a.ldv + (int64_t)h * a.vdim + cc] : 0.f;
        }
        rb = (tid < ct && !a.plain) ? a.beta[(int64_t)(first + t0 + tid) * a.ldbeta + h] : 0.f;
    };
    auto stage = [&](int b) {
#pragma unroll
        for (int j = 0; j < NL; j++) {
            const int i = tid + 256 * j, tt = i / DP, d = i % DP, at = (d & (DR_RS - 1)) * LDP + (d >> 4);   // row d = r + 16 u -> [r][u]
            sq[(b * CT + tt) * ROW + at] = rq[j];
            sk[(b * CT + tt) * ROW + at] = rk[j];
            sg[(b * CT + tt) * ROW + at] = rg[j];
        }
#pragma unroll
        for (int j = 0; j < NV; j++) {
            const int i = tid + 256 * j;
            if (i < CT * DR_VT) sv[b * CT * DR_VT + i] = rv[j];
        }
        if (tid < CT) sb[b * CT + tid] = rb;
    };
    request(0);
    stage(0);
    __syncthreads();
    int b = 0;
    for (int t0 = 0; t0 < count; t0 += CT, b ^= 1) {
        const int ct = min(CT, count - t0);
        const bool more = t0 + CT < count;
        if (more) request(t0 + CT);
        // The read-out is taken from the decayed memory: o = (gS)^T q + u (k . q), so the three column sums of a token, (gS)^T k,
        // (gS)^T q and k . q, are independent chains and the write S += k u^T leaves the critical path.  The LDS reads of the next
        // token are issued before the current one is worked on (two register sets, A and B).
        auto ld = [&](int tt, float (&kk)[DPT], float (&gg)[DPT], float (&qq)[DPT], float &bv, float &vv) {
#pragma unroll
            for (int u = 0; u < DPT; u += 4) {
                const float4 k4 = *reinterpret_cast<const float4 *>(sk + (b * CT + tt) * ROW + r * LDP + u);
                const float4 g4 = *reinterpret_cast<const float4 *>(sg + (b * CT + tt) * ROW + r * LDP + u);
                const float4 q4 = *reinterpret_cast<const float4 *>(sq + (b * CT + tt) * ROW + r * LDP + u);
                kk[u] = k4.x, kk[u + 1] = k4.y, kk[u + 2] = k4.z, kk[u + 3] = k4.w;
                gg[u] = g4.x, gg[u + 1] = g4.y, gg[u + 2] = g4.z, gg[u + 3] = g4.w;
                qq[u] = q4.x, qq[u + 1] = q4.y, qq[u + 2] = q4.z, qq[u + 3] = q4.w;
            }
            bv = sb[b * CT + tt];
            vv = sv[(b * CT + tt) * DR_VT + cl];
        };
        auto step = [&](int tt, const float (&kk)[DPT], const float (&gg)[DPT], const float (&qq)[DPT], float bv, float vv) {
            float pk = 0.f, pq = 0.f, kq = 0.f;
#pragma unroll
            for (int u = 0; u < DPT; u++) {
                S[u] *= gg[u];
                pk = fmaf(S[u], kk[u], pk);
                pq = fmaf(S[u], qq[u], pq);
                kq = fmaf(kk[u], qq[u], kq);
            }
            pk += vmx_dpp<VMX_DPP_XOR1>(pk), pq += vmx_dpp<VMX_DPP_XOR1>(pq), kq += vmx_dpp<VMX_DPP_XOR1>(kq);
            pk += vmx_dpp<VMX_DPP_XOR2>(pk), pq += vmx_dpp<VMX_DPP_XOR2>(pq), kq += vmx_dpp<VMX_DPP_XOR2>(kq);
            pk += vmx_dpp<VMX_DPP_HALF_MIRROR>(pk), pq += vmx_dpp<VMX_DPP_HALF_MIRROR>(pq), kq += vmx_dpp<VMX_DPP_HALF_MIRROR>(kq);
            pk += vmx_dpp<VMX_DPP_ROR8>(pk), pq += vmx_dpp<VMX_DPP_ROR8>(pq), kq += vmx_dpp<VMX_DPP_ROR8>(kq);
            const float uu = a.plain ? vv : bv * (vv - pk);
            if (r == 0 && c < a.vdim) a.o[(int64_t)(first + t0 + tt) * a.ldo + (int64_t)h * a.vdim + c] = fmaf(uu, kq, pq);
#pragma unroll
            for (int u = 0; u < DPT; u++) S[u] = fmaf(kk[u], uu, S[u]);
        };
        float kA[DPT], gA[DPT], qA[DPT], kB[DPT], gB[DPT], qB[DPT], bA, vA, bB = 0.f, vB = 0.f;
        ld(0, kA, gA, qA, bA, vA);
        for (int tt = 0; tt < ct; tt += 2) {
            if (tt + 1 < ct) ld(tt + 1, kB, gB, qB, bB, vB);
            step(tt, kA, gA, qA, bA, vA);
            if (tt + 1 < ct) {
                if (tt + 2 < ct) ld(tt + 2, kA, gA, qA, bA, vA);
                step(tt + 1, kB, gB, qB, bB, vB);
            }
        }
        if (more) stage(b ^ 1);
        __syncthreads();
    }
#pragma unroll
    for (int u = 0; u < DPT; u++) sp[(int64_t)u * 256] = S[u];
}

// y[t, h] = o[t, h] / sqrt(mean(o^2) + eps) * w * sigmoid(gate[t, h]) (gate_silu: * silu(gate[t, h])); one wave per (token, head);
// w bf16 [vdim] shared by heads (NULL: no gain)
__global__ __launch_bounds__(256) void head_rms_gate_kernel(void *__restrict__ y, int y_f32, const float *__restrict__ o, int64_t ldo,
                                                             const uint16_t *__restrict__ w, const float *__restrict__ gate, int64_t ldgate,
                                                             float eps, int rows, int heads, int vdim, int gate_silu) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    const int t = row / heads, h = row % heads;
    const float *src = o + (int64_t)t * ldo + (int64_t)h * vdim;
    float ss = 0.f;
    for (int i = lane; i < vdim; i += 64) ss = fmaf(src[i], src[i], ss);
    ss = vmx_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)vdim + eps);
    for (int i = lane; i < vdim; i += 64) {
        float v = src[i] * inv;
        if (w) v *= vmx_bf16_to_f32(w[i]);
        if (gate) {
            const float z = gate[(int64_t)t * ldgate + (int64_t)h * vdim + i];
            v *= gate_silu ? silu_f(z) : sigmoid_f(z);
        }
        const int64_t at = ((int64_t)t * heads + h) * vdim + i;
        if (y_f32) ((float *)y)[at] = v;
        else ((uint16_t *)y)[at] = vmx_f32_to_bf16(v);
    }
}

ConvArgs conv_args(const float *x, int64_t ldx, const uint16_t *taps, float *state, float *y, int64_t ldy, const int32_t *positions,
                   const int32_t *seq_ids, const int32_t *seq_starts, const int32_t *state_slots, int tokens, int channels, int n, int group,
                   int unit_groups, int scaled_groups, float unit_eps, float mul) {
    return ConvArgs{x, ldx, taps, state, y, ldy, positions, seq_ids, seq_starts, state_slots, tokens, channels, n, group, unit_groups,
                    scaled_groups, unit_eps, mul};
}

}  // namespace

extern "C" size_t vmx_short_conv_state_bytes(int slots, int channels, int taps) {
    return (size_t)slots * (size_t)(taps > 1 ? taps - 1 : 0) * channels * 4;
}

extern "C" int vmx_short_conv_silu(const float *x, int64_t ldx, const uint16_t *taps_bf16, float *state, float *y, int64_t ldy,
                                   const int32_t *positions, const int32_t *seq_ids, const int32_t *seq_starts, const int32_t *state_slots,
                                   int tokens, int channels, int taps, int unit_group, int unit_groups, int scaled_groups, float unit_eps,
                                   float scaled_mul, void *stream) {
    VMX_REQUIRE(x && taps_bf16 && y && positions && seq_ids && seq_starts && state_slots && (state || taps <= 1), "short_conv: null pointer");
    VMX_REQUIRE(channels >= 1 && taps >= 1 && ldx >= channels && ldy >= channels, "short_conv: bad sizes");
    VMX_REQUIRE(unit_groups >= 0 && scaled_groups >= 0 && scaled_groups <= unit_groups && (unit_groups == 0 || unit_group >= 1) &&
                    (int64_t)unit_groups * unit_group <= channels,
                "short_conv: bad unit-vector groups");
    if (tokens <= 0) return VMX_OK;
    const ConvArgs a = conv_args(x, ldx, taps_bf16, state, y, ldy, positions, seq_ids, seq_starts, state_slots, tokens, channels, taps, unit_group,
                                 unit_groups, scaled_groups, unit_eps, scaled_mul);
    const int runs = unit_groups + (channels - unit_groups * unit_group + 63) / 64;
    hipLaunchKernelGGL(short_conv_silu_kernel, dim3(tokens, (runs + 3) / 4), dim3(256), 0, vmx_stream(stream), a);
    VMX_CHECK_LAUNCH("short_conv_silu");
    return VMX_OK;
}

extern "C" int vmx_short_conv_state_update(const float *x, int64_t ldx, float *state, const int32_t *positions, const int32_t *seq_starts,
                                           const int32_t *state_slots, int num_seqs, int channels, int taps, void *stream) {
    VMX_REQUIRE(x && positions && seq_starts && state_slots && (state || taps <= 1), "short_conv_state_update: null pointer");
    if (num_seqs <= 0 || taps <= 1) return VMX_OK;
    const ConvArgs a = conv_args(x, ldx, nullptr, state, nullptr, 0, positions, nullptr, seq_starts, state_slots, 0, channels, taps, 1, 0, 0, 0.f, 1.f);
    hipLaunchKernelGGL(short_conv_state_kernel, dim3((channels + 255) / 256, num_seqs), dim3(256), 0, vmx_stream(stream), a, num_seqs);
    VMX_CHECK_LAUNCH("short_conv_state_update");
    return VMX_OK;
}

extern "C" int vmx_delta_rule_gates(float *g, int64_t ldg, const uint16_t *a_log_bf16, const uint16_t *dt_bias_bf16, float *beta,
                                    int64_t ldbeta, int tokens, int heads, int dim, void *stream) {
    VMX_REQUIRE(g && a_log_bf16 && dt_bias_bf16 && beta, "delta_rule_gates: null pointer");
    VMX_REQUIRE(heads >= 1 && dim >= 1 && ldg >= (int64_t)heads * dim && ldbeta >= heads, "delta_rule_gates: bad sizes");
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(delta_gates_kernel, dim3(tokens, (heads * dim + 255) / 256), dim3(256), 0, vmx_stream(stream), g, ldg, a_log_bf16,
                       dt_bias_bf16, beta, ldbeta, heads, dim);
    VMX_CHECK_LAUNCH("delta_rule_gates");
    return VMX_OK;
}

static int delta_dpt(int dim) { return dim <= 64 ? 4 : (dim <= 128 ? 8 : 16); }
static size_t delta_lds_bytes(int dpt) {
    const size_t ct = 128 / dpt, row = (size_t)DR_RS * (dpt == 4 ? 4 : dpt + 4);
    return (3 * 2 * ct * row + 2 * ct * DR_VT + 2 * ct) * 4;
}
template <int DPT> static int delta_launch(const DeltaArgs &a, dim3 grid, hipStream_t st) {
    static bool sized = false;   // more than 64 KiB of LDS has to be asked for once per kernel
    const size_t lds = delta_lds_bytes(DPT);
    if (!sized) {
        VMX_CHECK_HIP(hipFuncSetAttribute((const void *)gated_delta_rule_kernel<DPT>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        sized = true;
    }
    hipLaunchKernelGGL(gated_delta_rule_kernel<DPT>, grid, dim3(256), lds, st, a);
    return VMX_OK;
}

extern "C" size_t vmx_gated_delta_rule_state_bytes(int slots, int heads, int dim, int vdim) {
    const size_t tiles = (vdim + DR_VT - 1) / DR_VT;
    return (size_t)slots * heads * tiles * delta_dpt(dim) * 256 * 4;
}

extern "C" int vmx_gated_delta_rule(float *o, int64_t ldo, const float *q, int64_t ldq, const float *k, int64_t ldk, const float *v,
                                    int64_t ldv, const float *g, int64_t ldg, const float *beta, int64_t ldbeta, float *state,
                                    const int32_t *positions, const int32_t *seq_starts, const int32_t *state_slots, int num_seqs, int heads,
                                    int qk_heads, int dim, int vdim, void *stream) {
    VMX_REQUIRE(beta, "gated_delta_rule: null pointer");
    return vmx_matrix_memory_recurrence(o, ldo, q, ldq, 1.0f, k, ldk, v, ldv, g, ldg, 0, beta, ldbeta, state, positions, seq_starts, state_slots, num_seqs,
                                        heads, qk_heads, dim, vdim, stream);
}

extern "C" int vmx_sigmoid_root_decay(float *g, int64_t ldg, int tokens, int n, float tau, void *stream) {
    VMX_REQUIRE(g && n >= 1 && ldg >= n && tau > 0.f, "sigmoid_root_decay: bad arguments");
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(sigmoid_root_decay_kernel, dim3(tokens, (n + 255) / 256), dim3(256), 0, vmx_stream(stream), g, ldg, n, 1.0f / tau);
    VMX_CHECK_LAUNCH("sigmoid_root_decay");
    return VMX_OK;
}

extern "C" int vmx_matrix_memory_recurrence(float *o, int64_t ldo, const float *q, int64_t ldq, float q_mul, const float *k, int64_t ldk, const float *v,
                                            int64_t ldv, const float *g, int64_t ldg, int g_per_head, const float *beta, int64_t ldbeta,
                                            float *state, const int32_t *positions, const int32_t *seq_starts, const int32_t *state_slots,
                                            int num_seqs, int heads, int qk_heads, int dim, int vdim, void *stream) {
    VMX_REQUIRE(o && q && k && v && g && state && positions && seq_starts && state_slots, "matrix_memory_recurrence: null pointer");
    VMX_REQUIRE(heads >= 1 && qk_heads >= 1 && heads % qk_heads == 0, "matrix_memory_recurrence: %d heads do not share %d query/key heads evenly",
                heads, qk_heads);
    VMX_REQUIRE(dim >= 1 && dim <= 256 && vdim >= 1, "matrix_memory_recurrence: key size %d outside 1..256", dim);
    VMX_REQUIRE(ldg >= (g_per_head ? heads : (int64_t)heads * dim) || (g_per_head && ldg == 0), "matrix_memory_recurrence: bad decay row stride");
    if (num_seqs <= 0) return VMX_OK;
    const DeltaArgs a{q, k, v, g, beta, ldq, ldk, ldv, ldg, ldbeta, o, ldo, state, positions, seq_starts, state_slots, heads, qk_heads, dim, vdim,
                      g_per_head ? 1 : 0, beta ? 0 : 1, q_mul};
    const dim3 grid((vdim + DR_VT - 1) / DR_VT, heads, num_seqs);
    hipStream_t st = vmx_stream(stream);
    int rc;
    switch (delta_dpt(dim)) {
        case 4: rc = delta_launch<4>(a, grid, st); break;
        case 8: rc = delta_launch<8>(a, grid, st); break;
        default: rc = delta_launch<16>(a, grid, st); break;
    }
    if (rc) return rc;
    VMX_CHECK_LAUNCH("matrix_memory_recurrence");
    return VMX_OK;
}

extern "C" int vmx_head_rms_gate(void *y, int y_dtype, const float *o, int64_t ldo, const uint16_t *w_bf16, const float *gate, int64_t ldgate,
                                 float eps, int tokens, int heads, int vdim, void *stream) {
    VMX_REQUIRE(w_bf16, "head_rms_gate: null pointer");
    return vmx_head_rms_gate_ex(y, y_dtype, o, ldo, w_bf16, gate, ldgate, 0, eps, tokens, heads, vdim, stream);
}

extern "C" int vmx_head_rms_gate_ex(void *y, int y_dtype, const float *o, int64_t ldo, const uint16_t *w_bf16, const float *gate, int64_t ldgate,
                                    int gate_silu, float eps, int tokens, int heads, int vdim, void *stream) {
    VMX_REQUIRE(y && o, "head_rms_gate: null pointer");
    VMX_REQUIRE(y_dtype == VMX_F32 || y_dtype == VMX_BF16, "head_rms_gate: f32 or bf16 output");
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(head_rms_gate_kernel, dim3((tokens * heads + 3) / 4), dim3(256), 0, vmx_stream(stream), y, y_dtype == VMX_F32, o, ldo,
                       w_bf16, gate, ldgate, eps, tokens * heads, heads, vdim, gate_silu ? 1 : 0);
    VMX_CHECK_LAUNCH("head_rms_gate");
    return VMX_OK;
}
