// Linear layers over UNQUANTIZED bf16 weights for any shape: C[m, n] (op)= sum_k A[m, k] * W(n, k), f32 accumulation in ascending k.
// One argument block (VmxLinear, vmx_kernels.h) describes every variant the executors need:
//   * activations in f32 or bf16, output in f32 or bf16; weights addressed with two strides, so [N, K] (y = W x) and [K, N]
//     (y = W^T x, the absorbed key up-projection of latent attention) are the same kernel;
//   * blockIdx.z batches with element strides (one product per attention head);
//   * gathered activation rows and per-row-block weight matrices (experts of a mixture whose (token, slot) pairs were sorted into
//     blocks by vmx_moe_align_block_size);
//   * epilogues: plain store, squared ReLU, accumulate into an f32 residual stream, multiply by sigmoid(gate).
// Two kernels: `linear_fma_kernel` multiplies in true f32 on the vector ALU (the 32-bit mode of a model, and every product that
// must stay in 32 bits such as a router), `linear_mfma_kernel` rounds the activations to bf16 and runs v_mfma_f32_16x16x32_bf16.
// A row's result never depends on the other rows of the call: a row is summed in the same order whatever M is.
#include "vmx_kernels.h"

namespace {

__device__ __forceinline__ float ld_act(const void *A, int a_f32, int64_t i) {
    return a_f32 ? ((const float *)A)[i] : vmx_bf16_to_f32(((const uint16_t *)A)[i]);
}

__device__ __forceinline__ void linear_store(const VmxLinear &p, int z, int m, int n, float v) {
    if (p.epilogue == VMX_EP_RELU2) {
        const float r = fmaxf(v, 0.f);
        v = r * r;
    } else if (p.epilogue == VMX_EP_MUL_SIGMOID) {
        const float g = p.aux[(int64_t)m * p.ldaux + n + z * p.aux_bs];
        v *= 1.0f / (1.0f + expf(-g));
    }
    const int64_t o = (int64_t)m * p.ldc + n + z * p.c_bs;
    if (p.epilogue == VMX_EP_ADD_F32) ((float *)p.C)[o] += v;
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

}  // namespace

int vmx_linear_launch(const VmxLinear &p, hipStream_t st) {
    VMX_REQUIRE(p.A && p.W && p.C, "linear: null pointer");
    VMX_REQUIRE(p.M >= 0 && p.N > 0 && p.K > 0 && p.batch >= 1, "linear: bad shape M %d N %d K %d batch %d", p.M, p.N, p.K, p.batch);
    VMX_REQUIRE(p.epilogue != VMX_EP_ADD_F32 || p.c_f32, "linear: the accumulating epilogue needs an f32 output");
    VMX_REQUIRE(p.epilogue != VMX_EP_MUL_SIGMOID || p.aux, "linear: the gate epilogue needs its gate rows");
    VMX_REQUIRE(!p.block_expert || (p.total_rows && (p.block_rows == 16 || p.block_rows == 64)), "linear: expert blocks are 16 or 64 rows");
    VMX_REQUIRE(!p.row_ids || p.row_div >= 1, "linear: row_div must be positive");
    if (p.M == 0) return VMX_OK;
    const int bm = p.block_expert ? p.block_rows : (p.M <= 16 ? 16 : 64);
    dim3 grid((p.N + 63) / 64, (p.M + bm - 1) / bm, p.batch);
    if (bm == 16) hipLaunchKernelGGL(linear_fma_kernel<16>, grid, dim3(256), 0, st, p);
    else hipLaunchKernelGGL(linear_fma_kernel<64>, grid, dim3(256), 0, st, p);
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
