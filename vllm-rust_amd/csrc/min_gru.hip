// Minimal gated recurrent unit over packed steps: per channel, with gates that read only the current token,
//   z_t = sigmoid(zl_t);  c_t = u_t + 1/2 (u_t >= 0) | sigmoid(u_t) (u_t < 0);  S_t = (1 - z_t) S_(t-1) + z_t c_t;  y_t = S_t * silu(g_t)
// The state S lives in f32 in a slot per live sequence ([slots, width]); a sequence whose step starts at position 0 starts from
// zeros, so a slot is never cleared when it changes hands.  Everything here is f32.
//
// The recurrence is linear in S, S_t = a_t S_(t-1) + b_t, so a run of rows composes to one pair (A, B) = (prod a, the run's result
// from a zero start) and runs can be walked side by side: a workgroup owns 16 channels of one sequence and 64 strands (a wave
// holds four of them: 64-byte pieces of four rows per load), strand s the s-th 64th of the sequence's rows.  Pass 1: every strand
// composes its run; pass 2: it starts from the slot's state pushed through the pairs of the strands before it and walks its rows
// again, now storing y.  Steps whose runs are at most four rows long (decode) take the one-strand form: a thread per (sequence,
// channel), 256 channels a workgroup.  A row's result depends on where the strands' borders fall only by f32 rounding of the
// composition.
#include "vmx_kernels.h"

namespace {

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// <16 channels, 64 strands> for steps with prompt portions; <256, 1> when every sequence brings at most one row per strand anyway
// (decode steps: tokens - sequences + 1 bounds the longest run)
template <int GRU_CH, int GRU_STRANDS>
__global__ __launch_bounds__(GRU_CH * GRU_STRANDS) void min_gru_kernel(void *__restrict__ y, int y_f32, const float *__restrict__ zl, int64_t ldz,
                                                                   const float *__restrict__ u, int64_t ldu, const float *__restrict__ g,
                                                                   int64_t ldg, float *__restrict__ state, const int32_t *__restrict__ positions,
                                                                   const int32_t *__restrict__ seq_starts, const int32_t *__restrict__ state_slots,
                                                                   int width) {
    __shared__ float As[GRU_STRANDS][GRU_CH], Bs[GRU_STRANDS][GRU_CH];
    const int lane = threadIdx.x % GRU_CH, strand = threadIdx.x / GRU_CH;
    const int c = blockIdx.x * GRU_CH + lane, s = blockIdx.y;
    const int r0 = seq_starts[s], len = seq_starts[s + 1] - r0;
    if (len <= 0) return;   // the same for the whole workgroup
    const bool live = c < width;
    const int per = (len + GRU_STRANDS - 1) / GRU_STRANDS;
    const int a0 = min(len, strand * per), a1 = min(len, a0 + per);
    float A = 1.0f, B = 0.0f;
    if (live)
        for (int t = a0; t < a1; t++) {
            const int64_t r = r0 + t;
            const float z = sigmoid_f32(zl[r * ldz + c]), x = u[r * ldu + c];
            const float cand = x >= 0.f ? x + 0.5f : sigmoid_f32(x);
            A *= 1.0f - z;
            B = fmaf(1.0f - z, B, z * cand);
        }
    As[strand][lane] = A;
    Bs[strand][lane] = B;
    __syncthreads();
    if (!live) return;
    float *slot = state + (int64_t)state_slots[s] * width;
    float S = positions[r0] == 0 ? 0.0f : slot[c];
    for (int p = 0; p < strand; p++) S = fmaf(As[p][lane], S, Bs[p][lane]);
    for (int t = a0; t < a1; t++) {
        const int64_t r = r0 + t;
        const float z = sigmoid_f32(zl[r * ldz + c]), x = u[r * ldu + c];
        const float cand = x >= 0.f ? x + 0.5f : sigmoid_f32(x);
        S = fmaf(1.0f - z, S, z * cand);
        float o = S;
        if (g) {
            const float gv = g[r * ldg + c];
            o *= gv * sigmoid_f32(gv);
        }
        if (y_f32) ((float *)y)[r * width + c] = o;
        else ((uint16_t *)y)[r * width + c] = vmx_f32_to_bf16(o);
    }
    if (a1 == len && a0 < a1) slot[c] = S;   // the strand that holds the last row (exactly one: a0 < len = a1)
}

}  // namespace

extern "C" size_t vmx_min_gru_state_bytes(int slots, int width) { return (size_t)(slots > 0 ? slots : 0) * (width > 0 ? width : 0) * 4; }

extern "C" int vmx_min_gru(void *y, int y_dtype, const float *zl, int64_t ldz, const float *u, int64_t ldu, const float *g, int64_t ldg,
                           float *state, const int32_t *positions, const int32_t *seq_starts, const int32_t *state_slots, int num_seqs,
                           int tokens, int width, void *stream) {
    VMX_REQUIRE(y && zl && u && state && positions && seq_starts && state_slots, "min_gru: null pointer");
    VMX_REQUIRE(y_dtype == VMX_F32 || y_dtype == VMX_BF16, "min_gru: f32 or bf16 output");
    VMX_REQUIRE(width >= 1 && ldz >= width && ldu >= width && (!g || ldg >= width), "min_gru: bad width or row strides");
    VMX_REQUIRE(num_seqs >= 0 && num_seqs <= 65535, "min_gru: %d sequences in one step", num_seqs);
    if (num_seqs == 0 || tokens <= 0) return VMX_OK;
    hipStream_t st = vmx_stream(stream);
    if (tokens - num_seqs + 1 <= 4)   // no run longer than four rows
        hipLaunchKernelGGL((min_gru_kernel<256, 1>), dim3((width + 255) / 256, num_seqs), dim3(256), 0, st, y, y_dtype == VMX_F32, zl, ldz, u, ldu, g, ldg,
                           state, positions, seq_starts, state_slots, width);
    else
        hipLaunchKernelGGL((min_gru_kernel<16, 64>), dim3((width + 15) / 16, num_seqs), dim3(1024), 0, st, y, y_dtype == VMX_F32, zl, ldz, u, ldu, g, ldg,
                           state, positions, seq_starts, state_slots, width);
    VMX_CHECK_LAUNCH("min_gru");
    return VMX_OK;
}
