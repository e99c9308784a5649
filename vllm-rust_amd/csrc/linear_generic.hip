// Linear layers over UNQUANTIZED bf16 weights for any shape: C[m, n] (op)= sum_k A[m, k] * W(n, k), f32 accumulation in ascending k.
// One argument block (VmxLinear, vmx_kernels.h) describes every variant the executors need:
//   * activations in f32 or bf16, output in f32 or bf16; weights addressed with two strides, so [N, K] (y = W x) and [K, N]
//     (y = W^T x, the absorbed key up-projection of latent attention) are the same kernel;
//   * blockIdx.z batches with element strides (one product per attention head);
//   * gathered activation rows and per-row-block weight matrices (experts of a mixture whose (token, slot) pairs were sorted into
//     blocks by vmx_moe_align_block_size);
//   * an optional bf16 bias per output column, then an epilogue: plain store, squared ReLU, tanh-form GELU, accumulate into an
//     f32 residual stream, multiply by sigmoid(gate), or both of the last two (a gated residual update).
// Kernels: `linear_mfma_kernel` (64-row tiles for prompts and 64-row expert blocks; a staged 16-row form for shapes the streaming
// kernel does not take) and `linear_skinny_kernel` (up to 16 rows: decode steps and 16-row expert blocks, weights streamed once)
// round the activations to bf16 and run v_mfma_f32_16x16x32_bf16; `linear_fma_kernel` multiplies in true f32 on the vector ALU
// (the 32-bit mode of a model), `linear_fewcols_f32_kernel` does the same for a few output columns (router logits) with one
// kernel for every row count.  A row's result never depends on the other rows of the call: within a kernel a row is summed in
// the same order whatever M is; between the streaming and the tiled kernels the order differs (rounding-level differences).
#include "vmx_kernels.h"

namespace {

__device__ __forceinline__ float ld_act(const void *A, int a_f32, int64_t i) {
    return a_f32 ? ((const float *)A)[i] : vmx_bf16_to_f32(((const uint16_t *)A)[i]);
}

__device__ __forceinline__ void linear_store(const VmxLinear &p, int z, int m, int n, float v) {
    if (p.bias) v += vmx_bf16_to_f32(p.bias[n + z * p.bias_bs]);
    if (p.epilogue == VMX_EP_RELU2) {
        const float r = fmaxf(v, 0.f);
        v = r * r;
    } else if (p.epilogue == VMX_EP_GELU_TANH) {
        v = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
    } else if (p.epilogue == VMX_EP_MUL_SIGMOID || p.epilogue == VMX_EP_ADD_MUL_SIGMOID) {
        const float g = p.aux[(int64_t)m * p.ldaux + n + z * p.aux_bs];
        v *= 1.0f / (1.0f + expf(-g));
    }
    v *= p.out_scale;
    const int64_t o = (int64_t)m * p.ldc + n + z * p.c_bs;
    if (p.epilogue == VMX_EP_ADD_F32 || p.epilogue == VMX_EP_ADD_MUL_SIGMOID) ((float *)p.C)[o] += v;
    else if (p.c_f32) ((float *)p.C)[o] = v;
    else ((uint16_t *)p.C)[o] = vmx_f32_to_bf16(v);
}

// source row of output row m, or -1 for padding / out of range
__device__ __forceinline__ int64_t linear_src_row(const VmxLinear &p, int m) {
    if (m >= p.M) return -1;
    if (!p.row_ids) return m;
    const int r = p.row_ids[m];
    return (r < 0 || r >= p.row_limit) ? -1 : r / p.row_div;
}

// BM x 64 output tile per workgroup, 16 x 16 threads, (BM / 16) x 4 outputs per thread, 16-deep k steps through LDS.
template <int BM>
__global__ __launch_bounds__(256) void linear_fma_kernel(const VmxLinear p) {
    constexpr int BN = 64, BK = 16, TM = BM / 16, TN = 4;
    __shared__ float As[BK][BM + 1];
    __shared__ float Ws[BK][BN + 1];
    __shared__ int64_t rows[BM];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN, z = blockIdx.z;
    if (p.total_rows && m0 >= *p.total_rows) return;
    const uint16_t *W = p.W + z * p.w_bs;
    if (p.block_expert) W += (int64_t)p.block_expert[m0 / p.block_rows] * p.expert_stride;
    const int64_t a_off = z * p.a_bs;
    for (int i = tid; i < BM; i += 256) rows[i] = linear_src_row(p, m0 + i);
    __syncthreads();
    float acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = 0.f;
    const bool wk_fast = p.w_sk == 1;
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        for (int i = tid; i < BM * BK; i += 256) {
            const int m = i / BK, k = i % BK;
            const int64_t r = rows[m];
            As[k][m] = (r >= 0 && k0 + k < p.K) ? ld_act(p.A, p.a_f32, a_off + r * p.lda + k0 + k) : 0.f;
        }
        for (int i = tid; i < BN * BK; i += 256) {
            const int n = wk_fast ? i / BK : i % BN, k = wk_fast ? i % BK : i / BN;
            Ws[k][n] = (n0 + n < p.N && k0 + k < p.K) ? vmx_bf16_to_f32(W[(int64_t)(n0 + n) * p.w_sn + (int64_t)(k0 + k) * p.w_sk]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; k++) {
            float a[TM], w[TN];
#pragma unroll
            for (int i = 0; i < TM; i++) a[i] = As[k][ty * TM + i];
#pragma unroll
            for (int j = 0; j < TN; j++) w[j] = Ws[k][tx + 16 * j];
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
        const int m = m0 + ty * TM + i;
        if (m >= p.M || (p.row_ids && rows[ty * TM + i] < 0)) continue;
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int n = n0 + tx + 16 * j;
            if (n < p.N) linear_store(p, z, m, n, acc[i][j]);
        }
    }
}

// Matrix-core form: BM x 64 output tile, 64-deep k stages of bf16 in LDS (rows padded by 16 bytes), v_mfma_f32_16x16x32_bf16.
// BM = 64: wave w owns the 32 x 32 quadrant (w >> 1, w & 1) as 2 x 2 instruction tiles; BM = 16: wave w owns columns 16 w .. + 16.
// The next stage is requested into registers before the current one is multiplied.  An output element sums its k in the same
// order in both shapes, so a row's result does not depend on which shape its call took.
template <int BM>
__global__ __launch_bounds__(256) void linear_mfma_kernel(const VmxLinear p) {
    constexpr int BN = 64, BK = 64, LD = BK + 8, CH = BK / 8;   // CH: 8-element chunks per staged row
    constexpr int TI = BM == 64 ? 2 : 1, TJ = BM == 64 ? 2 : 1;
    constexpr int ACH = (BM * CH + 255) / 256, WCH = BN * CH / 256;
    __shared__ __align__(16) uint16_t As[BM * LD];
    __shared__ __align__(16) uint16_t Ws[BN * LD];
    __shared__ int64_t rows[BM];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN, z = blockIdx.z;
    if (p.total_rows && m0 >= *p.total_rows) return;
    const uint16_t *W = p.W + z * p.w_bs;
    if (p.block_expert) W += (int64_t)p.block_expert[m0 / p.block_rows] * p.expert_stride;
    const int64_t a_off = z * p.a_bs;
    for (int i = tid; i < BM; i += 256) rows[i] = linear_src_row(p, m0 + i);
    __syncthreads();
    // 16-byte loads need aligned rows: every row start and every chunk a multiple of 8 (bf16) elements
    const bool a_vec = (p.K & 7) == 0 && (p.lda & 7) == 0 && (a_off & 7) == 0 && ((uintptr_t)p.A & 31) == 0;
    const bool w_vec = p.w_sk == 1 && (p.K & 7) == 0 && (p.w_sn & 7) == 0 && (((uintptr_t)W) & 15) == 0;
    uint4 ar[ACH], wr[WCH];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int c = 0; c < ACH; c++) {
            const int idx = tid + 256 * c, m = idx / CH, k = k0 + 8 * (idx % CH);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (idx < BM * CH) {
                const int64_t r = rows[m];
                if (r >= 0 && k < p.K) {
                    const int64_t at = a_off + r * p.lda + k;
                    if (a_vec) {
                        if (p.a_f32) {
                            const float4 f0 = *reinterpret_cast<const float4 *>((const float *)p.A + at);
                            const float4 f1 = *reinterpret_cast<const float4 *>((const float *)p.A + at + 4);
                            const float f[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
                            v = vmx_pack16x8<false>(f);
                        } else {
                            v = *reinterpret_cast<const uint4 *>((const uint16_t *)p.A + at);
                        }
                    } else {
                        float f[8];
#pragma unroll
                        for (int e = 0; e < 8; e++) f[e] = k + e < p.K ? ld_act(p.A, p.a_f32, at + e) : 0.f;
                        v = vmx_pack16x8<false>(f);
                    }
                }
            }
            ar[c] = v;
        }
#pragma unroll
        for (int c = 0; c < WCH; c++) {
            const int idx = tid + 256 * c, n = n0 + idx / CH, k = k0 + 8 * (idx % CH);
            uint4 v = make_uint4(0, 0, 0, 0);
            if (n < p.N && k < p.K) {
                if (w_vec) {
                    v = *reinterpret_cast<const uint4 *>(W + (int64_t)n * p.w_sn + k);
                } else {
                    uint32_t h[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) h[e] = k + e < p.K ? W[(int64_t)n * p.w_sn + (int64_t)(k + e) * p.w_sk] : 0;
                    v = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
                }
            }
            wr[c] = v;
        }
    };
    auto stash = [&]() {
#pragma unroll
        for (int c = 0; c < ACH; c++) {
            const int idx = tid + 256 * c;
            if (idx < BM * CH) *reinterpret_cast<uint4 *>(As + (idx / CH) * LD + 8 * (idx % CH)) = ar[c];
        }
#pragma unroll
        for (int c = 0; c < WCH; c++) {
            const int idx = tid + 256 * c;
            *reinterpret_cast<uint4 *>(Ws + (idx / CH) * LD + 8 * (idx % CH)) = wr[c];
        }
    };
    vmx_f32x4 acc[TI][TJ];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < TJ; j++) acc[i][j] = vmx_f32x4{0.f, 0.f, 0.f, 0.f};
    const int wm = BM == 64 ? (wave >> 1) * 32 : 0, wn = BM == 64 ? (wave & 1) * 32 : wave * 16;
    const int fl = lane & 15, fg = lane >> 4;
    fetch(0);
    stash();
    __syncthreads();
    for (int k0 = 0; k0 < p.K; k0 += BK) {
        if (k0 + BK < p.K) fetch(k0 + BK);
#pragma unroll
        for (int s = 0; s < BK / 32; s++) {
            uint4 af[TI], wf[TJ];
#pragma unroll
            for (int i = 0; i < TI; i++) af[i] = *reinterpret_cast<const uint4 *>(As + (wm + 16 * i + fl) * LD + 32 * s + 8 * fg);
#pragma unroll
            for (int j = 0; j < TJ; j++) wf[j] = *reinterpret_cast<const uint4 *>(Ws + (wn + 16 * j + fl) * LD + 32 * s + 8 * fg);
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < TJ; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, af[i]), __builtin_bit_cast(vmx_bf16x8, wf[j]),
                                                                        acc[i][j], 0, 0, 0);
        }
        __syncthreads();
        if (k0 + BK < p.K) {
            stash();
            __syncthreads();
        }
    }
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int ml = wm + 16 * i + 4 * fg + r, m = m0 + ml;
            if (m >= p.M || (p.row_ids && rows[ml] < 0)) continue;
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int n = n0 + wn + 16 * j + fl;
                if (n < p.N) linear_store(p, z, m, n, acc[i][j][r]);
            }
        }
}

// Up to 16 rows (decode steps, 16-row expert blocks): the product is a stream over the weights.  A workgroup owns 16 output
// columns; its four waves split K in 128-deep blocks (wave w takes blocks w, w + 4, ...), lane (n, g) reads the 64 contiguous
// bytes W[n][128 b + 32 g ..] of a block straight from memory, two blocks ahead of the one being multiplied, and the activation
// fragment at the same k from the (cache-resident) rows; chunk j of both feeds MFMA step j -- the instruction only needs A and B
// to agree on which k sits where.  The four partial tiles are added in wave order through LDS.
__global__ __launch_bounds__(256) void linear_skinny_kernel(const VmxLinear p) {
    __shared__ float red[3][64][4];
    __shared__ int64_t rows[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fl = lane & 15, fg = lane >> 4;
    const int m0 = blockIdx.y * 16, n0 = blockIdx.x * 16, z = blockIdx.z;
    if (p.total_rows && m0 >= *p.total_rows) return;
    const uint16_t *W = p.W + z * p.w_bs;
    if (p.block_expert) W += (int64_t)p.block_expert[m0 / p.block_rows] * p.expert_stride;
    if (tid < 16) rows[tid] = linear_src_row(p, m0 + tid);
    __syncthreads();
    const int64_t ar = rows[fl];
    const int n = min(n0 + fl, p.N - 1);
    const uint16_t *wrow = W + (int64_t)n * p.w_sn;
    const int64_t a_at = z * p.a_bs + (ar < 0 ? 0 : ar) * p.lda;
    const int nblk = (p.K + 127) >> 7;
    auto load_w = [&](int b, uint4 (&w)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int k = 128 * b + 32 * fg + 8 * j;
            w[j] = k < p.K ? *reinterpret_cast<const uint4 *>(wrow + k) : make_uint4(0, 0, 0, 0);
        }
    };
    auto load_a = [&](int b, uint4 (&a)[4]) {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int k = 128 * b + 32 * fg + 8 * j;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (ar >= 0 && k < p.K) {
                if (p.a_f32) {
                    const float *src = (const float *)p.A + a_at + k;
                    const float4 f0 = *reinterpret_cast<const float4 *>(src), f1 = *reinterpret_cast<const float4 *>(src + 4);
                    const float f[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
                    v = vmx_pack16x8<false>(f);
                } else {
                    v = *reinterpret_cast<const uint4 *>((const uint16_t *)p.A + a_at + k);
                }
            }
            a[j] = v;
        }
    };
    vmx_f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    uint4 w0[4], w1[4], a0[4], a1[4];
    int b = wave;
    if (b < nblk) { load_w(b, w0); load_a(b, a0); }
    if (b + 4 < nblk) { load_w(b + 4, w1); load_a(b + 4, a1); }
    for (; b < nblk; b += 8) {
        uint4 wc[4], ac[4];
#pragma unroll
        for (int j = 0; j < 4; j++) wc[j] = w0[j], ac[j] = a0[j];
        if (b + 8 < nblk) { load_w(b + 8, w0); load_a(b + 8, a0); }
#pragma unroll
        for (int j = 0; j < 4; j++)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, ac[j]), __builtin_bit_cast(vmx_bf16x8, wc[j]), acc, 0, 0, 0);
        if (b + 4 < nblk) {
#pragma unroll
            for (int j = 0; j < 4; j++) wc[j] = w1[j], ac[j] = a1[j];
            if (b + 12 < nblk) { load_w(b + 12, w1); load_a(b + 12, a1); }
#pragma unroll
            for (int j = 0; j < 4; j++)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, ac[j]), __builtin_bit_cast(vmx_bf16x8, wc[j]), acc, 0, 0, 0);
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) red[wave - 1][lane][r] = acc[r];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float v = ((acc[r] + red[0][lane][r]) + red[1][lane][r]) + red[2][lane][r];
            const int ml = 4 * fg + r, m = m0 + ml;
            if (m < p.M && !(p.row_ids && rows[ml] < 0) && n0 + fl < p.N) linear_store(p, z, m, n0 + fl, v);
        }
    }
}

// A few output columns in true f32 (router logits): one workgroup per row and group of 16 columns; a thread walks its k with
// stride 256 over all 16 weight rows, then lanes, then waves are added in a fixed order.  Every row count takes this kernel, so
// a row's logits have the same bits in a prompt and in a decode step.
__global__ __launch_bounds__(256) void linear_fewcols_f32_kernel(const VmxLinear p) {
    __shared__ float red[4][16];
    const int m = blockIdx.x, n0 = blockIdx.y * 16, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    float acc[16];
#pragma unroll
    for (int e = 0; e < 16; e++) acc[e] = 0.f;
    for (int k = tid; k < p.K; k += 256) {
        const float x = ld_act(p.A, p.a_f32, (int64_t)m * p.lda + k);
#pragma unroll
        for (int e = 0; e < 16; e++) {
            const int n = min(n0 + e, p.N - 1);
            acc[e] = fmaf(x, vmx_bf16_to_f32(p.W[(int64_t)n * p.w_sn + k]), acc[e]);
        }
    }
#pragma unroll
    for (int e = 0; e < 16; e++) {
        const float v = vmx_wave_sum(acc[e]);
        if (lane == 0) red[wave][e] = v;
    }
    __syncthreads();
    if (tid < 16 && n0 + tid < p.N) linear_store(p, 0, m, n0 + tid, (red[0][tid] + red[1][tid]) + (red[2][tid] + red[3][tid]));
}

}  // namespace

int vmx_linear_launch(const VmxLinear &p, hipStream_t st) {
    VMX_REQUIRE(p.A && p.W && p.C, "linear: null pointer");
    VMX_REQUIRE(p.M >= 0 && p.N > 0 && p.K > 0 && p.batch >= 1, "linear: bad shape M %d N %d K %d batch %d", p.M, p.N, p.K, p.batch);
    VMX_REQUIRE((p.epilogue != VMX_EP_ADD_F32 && p.epilogue != VMX_EP_ADD_MUL_SIGMOID) || p.c_f32, "linear: the accumulating epilogues need an f32 output");
    VMX_REQUIRE((p.epilogue != VMX_EP_MUL_SIGMOID && p.epilogue != VMX_EP_ADD_MUL_SIGMOID) || p.aux, "linear: the gate epilogues need their gate rows");
    VMX_REQUIRE(!p.block_expert || (p.total_rows && (p.block_rows == 16 || p.block_rows == 64)), "linear: expert blocks are 16 or 64 rows");
    VMX_REQUIRE(!p.row_ids || p.row_div >= 1, "linear: row_div must be positive");
    if (p.M == 0) return VMX_OK;
    const bool plain = !p.row_ids && !p.block_expert && p.batch == 1 && p.w_sk == 1;
    if (p.exact && plain && p.N <= 256) {
        hipLaunchKernelGGL(linear_fewcols_f32_kernel, dim3(p.M, (p.N + 15) / 16), dim3(256), 0, st, p);
        VMX_CHECK_LAUNCH("linear (few columns)");
        return VMX_OK;
    }
    const int bm = p.block_expert ? p.block_rows : (p.M <= 16 ? 16 : 64);
    dim3 grid((p.N + 63) / 64, (p.M + bm - 1) / bm, p.batch);
    if (p.exact) {
        if (bm == 16) hipLaunchKernelGGL(linear_fma_kernel<16>, grid, dim3(256), 0, st, p);
        else hipLaunchKernelGGL(linear_fma_kernel<64>, grid, dim3(256), 0, st, p);
    } else {
        // 16-byte loads straight from the operands: whole 8-element chunks, aligned rows
        const bool direct = p.w_sk == 1 && p.K % 8 == 0 && p.w_sn % 8 == 0 && p.lda % 8 == 0 && p.a_bs % 8 == 0 && p.w_bs % 8 == 0 &&
                            p.expert_stride % 8 == 0 && ((uintptr_t)p.W & 15) == 0 && ((uintptr_t)p.A & 31) == 0;
        if (bm == 16 && direct) {
            grid.x = (p.N + 15) / 16;
            hipLaunchKernelGGL(linear_skinny_kernel, grid, dim3(256), 0, st, p);
        } else if (bm == 16) hipLaunchKernelGGL(linear_mfma_kernel<16>, grid, dim3(256), 0, st, p);
        else hipLaunchKernelGGL(linear_mfma_kernel<64>, grid, dim3(256), 0, st, p);
    }
    VMX_CHECK_LAUNCH("linear");
    return VMX_OK;
}

extern "C" int vmx_linear_bf16w(void *y, int y_dtype, const void *x, int x_dtype, const uint16_t *w, int M, int N, int K, int exact,
                                void *stream) {
    VMX_REQUIRE((y_dtype == VMX_F32 || y_dtype == VMX_BF16) && (x_dtype == VMX_F32 || x_dtype == VMX_BF16), "linear_bf16w: f32 or bf16 rows");
    VmxLinear p;
    p.A = x, p.a_f32 = x_dtype == VMX_F32, p.lda = K;
    p.W = w, p.w_sn = K, p.w_sk = 1;
    p.C = y, p.c_f32 = y_dtype == VMX_F32, p.ldc = N;
    p.M = M, p.N = N, p.K = K, p.exact = exact;
    return vmx_linear_launch(p, vmx_stream(stream));
}
