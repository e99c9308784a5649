// Routing of a mixture of experts on gfx950: the router's top-k selection (softmax or sigmoid scores, or softmax with
// group-limited choice) and the token -> expert alignment that sorts (token, slot) pairs into expert blocks.
// Semantics: crates/core/kernels/topk_softmax.cu:63-311 (softmax with expf, max-subtracted; k rounds of argmax, ties -> smaller
// index; optional renormalisation by the selected sum) and crates/core/kernels/fused_moe_align.cu:34-278 (moe_align_block_size).
// Sigmoid scores (vmx_topk_sigmoid): every expert's logit goes through the logistic function by itself; same selection.
#include "vmx_kernels.h"
#include <float.h>

namespace {

__device__ __forceinline__ float rb(float v) { return vmx_bf16_to_f32(vmx_f32_to_bf16(v)); }

// One wave per token; lane l holds experts l, l+64, ... (up to 4 per lane: E <= 256).
template <bool BF16_IN>
__global__ __launch_bounds__(256) void topk_softmax_kernel(const void *__restrict__ logits, float *__restrict__ w_out,
                                                            int32_t *__restrict__ id_out, int tokens, int E, int k, int renorm,
                                                            int round_probs_bf16, int sigmoid_scores) {
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (t >= tokens) return;
    float v[4];
    float mx = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = lane + 64 * j;
        v[j] = -FLT_MAX;
        if (e < E) v[j] = BF16_IN ? vmx_bf16_to_f32(((const uint16_t *)logits)[(int64_t)t * E + e]) : ((const float *)logits)[(int64_t)t * E + e];
        mx = fmaxf(mx, v[j]);
    }
    if (sigmoid_scores) {
        // every expert scored by itself, no sum over the experts: the logistic function keeps the order, so the choice is made on
        // the logits (where saturated scores would tie) and the chosen ones become scores as they are written
    } else {
        mx = vmx_wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[j] = (lane + 64 * j < E) ? expf(v[j] - mx) : 0.f;
            sum += v[j];
        }
        sum = vmx_wave_sum(sum);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[j] = (lane + 64 * j < E) ? v[j] / sum : -FLT_MAX;
            if (round_probs_bf16 && lane + 64 * j < E) v[j] = rb(v[j]);
        }
    }
    float selected = 0.f;
    for (int ki = 0; ki < k; ki++) {
        // key: larger value first, then smaller index
        float bv = -FLT_MAX;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int e = lane + 64 * j;
            if (e < E && (v[j] > bv)) { bv = v[j]; bi = e; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = vmx_lane_xor_m(bv, off);
            const int oi = vmx_lane_xor_m(bi, off);
            if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
        }
        if (sigmoid_scores) bv = 1.0f / (1.0f + expf(-bv));
        if (lane == 0) { w_out[(int64_t)t * k + ki] = bv; id_out[(int64_t)t * k + ki] = bi; }
        selected += bv;
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (lane + 64 * j == bi) v[j] = -FLT_MAX;
    }
    if (renorm && lane == 0) {
        const float f = selected > 0.f ? 1.0f / selected : 1.0f;
        for (int ki = 0; ki < k; ki++) w_out[(int64_t)t * k + ki] *= f;
    }
}

// (value, index) of the wave's largest value, ties to the smaller index; every lane ends with the same pair.  The six exchange
// steps are spelled out so that each is a DPP / permlane operation with a compile-time pattern.
template <int M> __device__ __forceinline__ void argmax_step(float &bv, int &bi) {
    const float ov = vmx_lane_xor<M>(bv);
    const int oi = vmx_lane_xor<M>(bi);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}
__device__ __forceinline__ void wave_argmax(float &bv, int &bi) {
    argmax_step<32>(bv, bi);
    argmax_step<16>(bv, bi);
    argmax_step<8>(bv, bi);
    argmax_step<4>(bv, bi);
    argmax_step<2>(bv, bi);
    argmax_step<1>(bv, bi);
}

// Router with group-limited selection: softmax over all experts; the experts form `groups` equal runs of neighbours, a group's
// score is its largest probability, and only experts of the `keep` best groups can be chosen; then k rounds of argmax (ties ->
// smaller index) over what is left.  Weights: the chosen probabilities divided by (their sum + 1e-20), times `scale`.
// One wave per token; lane l holds experts (and groups) l, l + 64, ...: E <= 256.
__global__ __launch_bounds__(256) void grouped_topk_router_kernel(const float *__restrict__ logits, float *__restrict__ w_out,
                                                                   int32_t *__restrict__ id_out, int tokens, int E, int k, int groups,
                                                                   int keep, float scale) {
    __shared__ float sc[4][256];
    __shared__ int32_t ok[4][256];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, t = blockIdx.x * 4 + wave;
    if (t >= tokens) return;   // no workgroup-wide barrier below: a wave only exchanges with itself
    float v[4];
    float mx = -FLT_MAX;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = lane + 64 * j;
        v[j] = e < E ? logits[(int64_t)t * E + e] : -FLT_MAX;
        mx = fmaxf(mx, v[j]);
    }
    mx = vmx_wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v[j] = (lane + 64 * j < E) ? expf(v[j] - mx) : 0.f;
        sum += v[j];
    }
    sum = vmx_wave_sum(sum);
#pragma unroll
    for (int j = 0; j < 4; j++) v[j] = (lane + 64 * j < E) ? v[j] / sum : -FLT_MAX;
    if (groups > 1 && keep < groups) {
        const int gs = E / groups;
#pragma unroll
        for (int j = 0; j < 4; j++) sc[wave][lane + 64 * j] = v[j];
        __builtin_amdgcn_wave_barrier();
        float gv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int g = lane + 64 * j;
            gv[j] = -FLT_MAX;
            if (g < groups)
                for (int i = 0; i < gs; i++) gv[j] = fmaxf(gv[j], sc[wave][g * gs + i]);
            ok[wave][g] = 0;
        }
        __builtin_amdgcn_wave_barrier();
        for (int r = 0; r < keep; r++) {
            float bv = -FLT_MAX;
            int bi = 0x7fffffff;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int g = lane + 64 * j;
                if (g < groups && gv[j] > bv) { bv = gv[j]; bi = g; }
            }
            wave_argmax(bv, bi);
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (lane + 64 * j == bi) { gv[j] = -FLT_MAX; ok[wave][bi] = 1; }
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int e = lane + 64 * j;
            if (e < E && !ok[wave][e / gs]) v[j] = -FLT_MAX;
        }
    }
    float selected = 0.f;
    for (int ki = 0; ki < k; ki++) {
        float bv = -FLT_MAX;
        int bi = 0x7fffffff;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int e = lane + 64 * j;
            if (e < E && v[j] > bv) { bv = v[j]; bi = e; }
        }
        wave_argmax(bv, bi);
        if (lane == 0) { w_out[(int64_t)t * k + ki] = bv; id_out[(int64_t)t * k + ki] = bi; }
        selected += bv;
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (lane + 64 * j == bi) v[j] = -FLT_MAX;
    }
    if (lane == 0) {
        const float f = scale / (selected + 1e-20f);
        for (int ki = 0; ki < k; ki++) w_out[(int64_t)t * k + ki] *= f;
    }
}

// Single workgroup.  sorted_token_ids: per expert, the flattened (token*k + slot) indices routed to it in
// ascending order, each expert's run padded to a multiple of block_size with `numel`; expert_ids: the
// expert of each block; total_tokens_post_pad[0] = padded length.
__global__ __launch_bounds__(256) void moe_align_kernel(const int32_t *__restrict__ topk_ids, int32_t *__restrict__ sorted,
                                                         int32_t *__restrict__ expert_ids, int32_t *__restrict__ total_post_pad,
                                                         int numel, int E, int block_size, int sorted_capacity) {
    extern __shared__ int32_t sh[];  // counts[E] | offsets[E+1]
    int32_t *counts = sh, *offs = sh + E;
    for (int e = threadIdx.x; e < E; e += 256) counts[e] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < numel; i += 256) {
        const int e = topk_ids[i];
        if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        for (int e = 0; e < E; e++) {
            offs[e] = acc;
            acc += (counts[e] + block_size - 1) / block_size * block_size;
        }
        offs[E] = acc;
        total_post_pad[0] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < sorted_capacity; i += 256) sorted[i] = numel;
    for (int b = threadIdx.x; b < offs[E] / block_size; b += 256) {
        int e = 0;
        while (e + 1 < E && offs[e + 1] <= b * block_size) e++;
        expert_ids[b] = e;
    }
    __syncthreads();
    // stable placement: thread e walks the ids in order (numel is small on the decode path)
    for (int e = threadIdx.x; e < E; e += 256) {
        int pos = offs[e];
        for (int i = 0; i < numel; i++)
            if (topk_ids[i] == e) sorted[pos++] = i;
    }
}

// The same result for up to 256 experts in O(numel / 1024) steps of one 1024-thread workgroup (the form above walks all ids once
// per expert): histogram with LDS atomics, serial prefix over the experts, then the ids in rounds of 1024 -- inside a wave the
// rank of an id among the earlier lanes with the same expert comes from ballots (one per distinct expert present in the wave),
// across the 16 waves from per-(wave, expert) counts in LDS -- so that an expert's indices still ascend.  One workgroup on
// purpose: the sort is a few microseconds in front of GEMMs that stream the experts, and a multi-workgroup form would cost
// two more dependent launches.
__global__ __launch_bounds__(1024) void moe_align_fast_kernel(const int32_t *__restrict__ topk_ids, int32_t *__restrict__ sorted,
                                                               int32_t *__restrict__ expert_ids, int32_t *__restrict__ total_post_pad,
                                                               int numel, int E, int block_size, int sorted_capacity) {
    extern __shared__ int32_t sh[];   // counts[E] | offs[E + 1] | cursor[E] | wave_cnt[16][E]
    int32_t *counts = sh, *offs = sh + E, *cursor = sh + 2 * E + 1, *wave_cnt = sh + 3 * E + 1;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int e = tid; e < E; e += 1024) counts[e] = 0;
    for (int i = tid; i < 16 * E; i += 1024) wave_cnt[i] = 0;
    __syncthreads();
    for (int i = tid; i < numel; i += 1024) {
        const int e = topk_ids[i];
        if (e >= 0 && e < E) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int acc = 0;
        for (int e = 0; e < E; e++) {
            offs[e] = acc;
            cursor[e] = acc;
            acc += (counts[e] + block_size - 1) / block_size * block_size;
        }
        offs[E] = acc;
        total_post_pad[0] = acc;
    }
    __syncthreads();
    for (int i = tid; i < sorted_capacity; i += 1024) sorted[i] = numel;
    for (int b = tid; b < offs[E] / block_size; b += 1024) {
        int lo = 0, hi = E - 1;   // the last expert whose run starts at or before this block (it is the one with rows there:
        while (lo < hi) {         // an empty expert shares its start with its successor, which is then the later one)
            const int mid = (lo + hi + 1) >> 1;
            if (offs[mid] <= b * block_size) lo = mid;
            else hi = mid - 1;
        }
        expert_ids[b] = lo;
    }
    __syncthreads();   // the padding fill is ordered before the placement below
    for (int base = 0; base < numel; base += 1024) {
        const int i = base + tid;
        const int e = i < numel ? topk_ids[i] : -1;
        const bool valid = e >= 0 && e < E;
        int rank = 0;
        unsigned long long remaining = __ballot(valid);
        while (remaining) {   // wave-uniform: one pass per distinct expert among this wave's ids
            const int leader = __ffsll((long long)remaining) - 1;
            const int le = __shfl(e, leader, 64);
            const unsigned long long mask = __ballot(valid && e == le);
            if (valid && e == le) rank = __popcll(mask & ((1ull << lane) - 1ull));
            if (lane == leader) wave_cnt[wave * E + le] = __popcll(mask);
            remaining &= ~mask;
        }
        __syncthreads();
        if (valid) {
            int before = 0;
            for (int w = 0; w < wave; w++) before += wave_cnt[w * E + e];
            sorted[cursor[e] + before + rank] = i;
        }
        __syncthreads();
        for (int ee = tid; ee < E; ee += 1024) {
            int tot = 0;
            for (int w = 0; w < 16; w++) {
                tot += wave_cnt[w * E + ee];
                wave_cnt[w * E + ee] = 0;
            }
            cursor[ee] += tot;
        }
        __syncthreads();
    }
}

}  // namespace

static int topk_scores(const void *logits, int logits_dtype, float *topk_weights, int32_t *topk_ids, int tokens, int num_experts, int k,
                       int renormalize, int round_probs_bf16, int sigmoid_scores, void *stream);

extern "C" int vmx_topk_softmax(const void *logits, int logits_dtype, float *topk_weights, int32_t *topk_ids, int tokens,
                                int num_experts, int k, int renormalize, int round_probs_bf16, void *stream) {
    return topk_scores(logits, logits_dtype, topk_weights, topk_ids, tokens, num_experts, k, renormalize, round_probs_bf16, 0, stream);
}

extern "C" int vmx_topk_sigmoid(const float *logits, float *topk_weights, int32_t *topk_ids, int tokens, int num_experts, int k,
                                int renormalize, void *stream) {
    return topk_scores(logits, VMX_F32, topk_weights, topk_ids, tokens, num_experts, k, renormalize, 0, 1, stream);
}

static int topk_scores(const void *logits, int logits_dtype, float *topk_weights, int32_t *topk_ids, int tokens, int num_experts, int k,
                       int renormalize, int round_probs_bf16, int sigmoid_scores, void *stream) {
    VMX_REQUIRE(logits && topk_weights && topk_ids, "topk_softmax: null pointer");
    VMX_REQUIRE(logits_dtype == VMX_F32 || logits_dtype == VMX_BF16, "topk_softmax: logits dtype must be f32 or bf16");
    VMX_REQUIRE(num_experts >= 1 && num_experts <= 256, "topk_softmax: num_experts (%d) must be in 1..256", num_experts);
    VMX_REQUIRE(k >= 1 && k <= num_experts, "topk_softmax: k (%d) must be in 1..num_experts", k);
    if (tokens <= 0) return VMX_OK;
    const dim3 grid((tokens + 3) / 4), block(256);
    if (logits_dtype == VMX_BF16)
        hipLaunchKernelGGL(topk_softmax_kernel<true>, grid, block, 0, vmx_stream(stream), logits, topk_weights, topk_ids, tokens, num_experts,
                           k, renormalize, round_probs_bf16, sigmoid_scores);
    else
        hipLaunchKernelGGL(topk_softmax_kernel<false>, grid, block, 0, vmx_stream(stream), logits, topk_weights, topk_ids, tokens, num_experts,
                           k, renormalize, round_probs_bf16, sigmoid_scores);
    VMX_CHECK_LAUNCH("topk_softmax");
    return VMX_OK;
}

extern "C" int vmx_grouped_topk_router(const float *logits, float *topk_weights, int32_t *topk_ids, int tokens, int num_experts, int k,
                                       int groups, int keep_groups, float scale, void *stream) {
    VMX_REQUIRE(logits && topk_weights && topk_ids, "grouped_topk_router: null pointer");
    VMX_REQUIRE(num_experts >= 1 && num_experts <= 256, "grouped_topk_router: num_experts (%d) must be in 1..256", num_experts);
    VMX_REQUIRE(groups >= 1 && num_experts % groups == 0, "grouped_topk_router: %d experts do not form %d equal groups", num_experts, groups);
    VMX_REQUIRE(keep_groups >= 1 && keep_groups <= groups, "grouped_topk_router: keep_groups (%d) must be in 1..groups", keep_groups);
    VMX_REQUIRE(k >= 1 && k <= keep_groups * (num_experts / groups), "grouped_topk_router: k (%d) exceeds the experts of the kept groups", k);
    if (tokens <= 0) return VMX_OK;
    hipLaunchKernelGGL(grouped_topk_router_kernel, dim3((tokens + 3) / 4), dim3(256), 0, vmx_stream(stream), logits, topk_weights, topk_ids,
                       tokens, num_experts, k, groups, keep_groups, scale);
    VMX_CHECK_LAUNCH("grouped_topk_router");
    return VMX_OK;
}

extern "C" int vmx_moe_align_block_size(const int32_t *topk_ids, int32_t *sorted_token_ids, int32_t *expert_ids,
                                        int32_t *total_tokens_post_pad, int numel, int num_experts, int block_size,
                                        int sorted_capacity, void *stream) {
    VMX_REQUIRE(topk_ids && sorted_token_ids && expert_ids && total_tokens_post_pad, "moe_align_block_size: null pointer");
    VMX_REQUIRE(numel >= 0 && num_experts >= 1 && num_experts <= 1024 && block_size >= 1, "moe_align_block_size: bad arguments");
    VMX_REQUIRE(sorted_capacity >= numel + num_experts * (block_size - 1), "moe_align_block_size: sorted_token_ids capacity %d too small",
                sorted_capacity);
    if (num_experts <= 256)
        hipLaunchKernelGGL(moe_align_fast_kernel, dim3(1), dim3(1024), (19 * num_experts + 1) * sizeof(int32_t), vmx_stream(stream), topk_ids,
                           sorted_token_ids, expert_ids, total_tokens_post_pad, numel, num_experts, block_size, sorted_capacity);
    else
        hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(256), (2 * num_experts + 1) * sizeof(int32_t), vmx_stream(stream), topk_ids,
                           sorted_token_ids, expert_ids, total_tokens_post_pad, numel, num_experts, block_size, sorted_capacity);
    VMX_CHECK_LAUNCH("moe_align_block_size");
    return VMX_OK;
}
