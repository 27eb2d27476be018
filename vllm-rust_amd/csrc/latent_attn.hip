// Latent attention over a paged cache of compressed keys/values.
//
// A token's cache row is [c | k_rot]: the RMS-normed latent c (kv_rank values) from which every head's unrotated key and value
// are linear maps (k_h = U_h c, v_h = V_h c), and one rotated key part (rot_dim values) shared by all heads.  The up-projections
// are never applied to the cache: with qa_h = U_h^T q_h (done by the caller as a batched product) the score of head h against
// key j is (qa_h . c_j + qr_h . k_rot_j) * scale, and the head's output is V_h (sum_j p_j c_j), so the kernel here works in the
// latent space -- every head reads the same cache rows -- and the caller applies V_h to its result.
//
// Parameters rather than constants: window (position i sees j with 0 <= i - j < window; 0 = unbounded causal), an optional
// per-head sink logit (a key-less term exp(sink_h) in the softmax denominator, not scaled), the rotation (interleaved pairs
// (2i, 2i+1) of the first rot_dims dimensions, angle = position * inv_freq[i]), sizes, cache element type (bf16 / f32).
// Scores, softmax, the weighted sum, norms and angles are f32.  Queries are packed: token t belongs to sequence seq_ids[t] at
// position positions[t], so prompts of different lengths, prompt portions and single decode tokens are the same launch, and a
// token's result depends only on its own query and the cache rows of its window.
#include "vmx_kernels.h"
#include <float.h>

namespace {

template <bool F32> __device__ __forceinline__ float ld_cache(const void *c, int64_t i) {
    if constexpr (F32) return ((const float *)c)[i];
    else return vmx_bf16_to_f32(((const uint16_t *)c)[i]);
}
template <bool F32> __device__ __forceinline__ void st_cache(void *c, int64_t i, float v) {
    if constexpr (F32) ((float *)c)[i] = v;
    else ((uint16_t *)c)[i] = vmx_f32_to_bf16(v);
}

// One workgroup per token: c = rms_norm(dkv[:R]) * w, k_rot = rotate(dkv[R:]) -> cache row `slot`; rotate(q_h[dim:]) -> q_rot.
template <bool F32>
__global__ __launch_bounds__(256) void latent_prepare_kernel(const float *__restrict__ fused, int64_t ldf, int q_off, int dkv_off,
                                                              const uint16_t *__restrict__ norm_w, float eps,
                                                              const float *__restrict__ inv_freq, int rot_dims,
                                                              const int32_t *__restrict__ positions, const int32_t *__restrict__ slots,
                                                              void *__restrict__ cache, float *__restrict__ q_rot, int H, int dim, int rd,
                                                              int R) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const float *row = fused + (int64_t)t * ldf;
    const float pos = (float)positions[t];
    const int64_t slot = slots[t];
    float ss = 0.f;
    for (int i = tid; i < R; i += 256) {
        const float v = row[dkv_off + i];
        ss += v * v;
    }
    ss = vmx_block_sum_256(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)R + eps);
    void *crow = cache;
    const int64_t cbase = slot * (R + rd);
    if (slot >= 0) {
        for (int i = tid; i < R; i += 256) st_cache<F32>(crow, cbase + i, row[dkv_off + i] * inv * vmx_bf16_to_f32(norm_w[i]));
    }
    // rotations: work item = (vector v, pair i); vector 0 is the shared key part, vector 1 + h the rotated part of head h's query
    const int half = rot_dims >> 1;
    for (int w = tid; w < (H + 1) * half; w += 256) {
        const int v = w / half, i = w % half;
        float sn, cs;
        sincosf(pos * inv_freq[i], &sn, &cs);
        const float *src = v == 0 ? row + dkv_off + R : row + q_off + (int64_t)(v - 1) * (dim + rd) + dim;
        const float a = src[2 * i], b = src[2 * i + 1];
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        if (v == 0) {
            if (slot >= 0) {
                st_cache<F32>(crow, cbase + R + 2 * i, ra);
                st_cache<F32>(crow, cbase + R + 2 * i + 1, rb);
            }
        } else {
            float *dst = q_rot + ((int64_t)t * H + (v - 1)) * rd;
            dst[2 * i] = ra;
            dst[2 * i + 1] = rb;
        }
    }
    // dimensions past rot_dims pass unchanged
    for (int w = tid; w < (H + 1) * (rd - rot_dims); w += 256) {
        const int v = w / (rd - rot_dims), i = rot_dims + w % (rd - rot_dims);
        if (v == 0) {
            if (slot >= 0) st_cache<F32>(crow, cbase + R + i, row[dkv_off + R + i]);
        } else {
            q_rot[((int64_t)t * H + (v - 1)) * rd + i] = row[q_off + (int64_t)(v - 1) * (dim + rd) + dim + i];
        }
    }
}

// One workgroup per (head, token).  Keys are walked 256 at a time: thread i scores key i of the chunk (a whole cache row against
// the query held in LDS), the chunk's maximum and sum update the running softmax, then wave w adds keys w, w + 4, ... of the chunk
// into its lanes' latent dimensions; the four waves are summed at the end.
template <bool F32>
__global__ __launch_bounds__(256) void latent_attn_kernel(float *__restrict__ out, const float *__restrict__ q_abs,
                                                           const float *__restrict__ q_rot, const void *__restrict__ cache,
                                                           const int32_t *__restrict__ block_tables, int max_blocks,
                                                           const int32_t *__restrict__ seq_ids, const int32_t *__restrict__ positions,
                                                           const uint16_t *__restrict__ sink, float scale, int window, int H, int R, int rd,
                                                           int block_size) {
    extern __shared__ float sm[];
    const int RW = R + rd;
    float *qs = sm;                 // [R + rd]
    float *ps = qs + RW;            // [256]
    int32_t *ks = (int32_t *)(ps + 256);   // [256] cache slots of the chunk's keys
    float *red = (float *)(ks + 256);      // [8]
    float *part = red + 8;          // [4][R]
    const int h = blockIdx.x, t = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pos = positions[t];
    const int32_t *bt = block_tables + (int64_t)seq_ids[t] * max_blocks;
    const int lo = window > 0 ? max(0, pos - window + 1) : 0;
    const int n = pos - lo + 1;
    for (int i = tid; i < R; i += 256) qs[i] = q_abs[((int64_t)t * H + h) * R + i];
    for (int i = tid; i < rd; i += 256) qs[R + i] = q_rot[((int64_t)t * H + h) * rd + i];
    constexpr int MAXD = 8;         // latent dimensions per lane: R <= 512
    float acc[MAXD];
#pragma unroll
    for (int i = 0; i < MAXD; i++) acc[i] = 0.f;
    // the sink enters as a key-less term: running maximum m = sink, running sum l = exp(sink - m) = 1
    float m = sink ? vmx_bf16_to_f32(sink[h]) : -FLT_MAX, l = sink ? 1.f : 0.f;
    __syncthreads();
    for (int c0 = 0; c0 < n; c0 += 256) {
        const bool valid = c0 + tid < n;
        float s = -FLT_MAX;
        if (valid) {
            const int j = lo + c0 + tid;
            const int slot = bt[j / block_size] * block_size + j % block_size;
            ks[tid] = slot;
            const int64_t base = (int64_t)slot * RW;
            float d = 0.f;
            if constexpr (!F32) {
                if ((RW & 7) == 0) {
                    const uint4 *r8 = reinterpret_cast<const uint4 *>((const uint16_t *)cache + base);
                    for (int i = 0; i < (RW >> 3); i++) {
                        float f[8];
                        vmx_unpack16x8<false>(r8[i], f);
#pragma unroll
                        for (int e = 0; e < 8; e++) d = fmaf(qs[8 * i + e], f[e], d);
                    }
                } else {
                    for (int i = 0; i < RW; i++) d = fmaf(qs[i], ld_cache<F32>(cache, base + i), d);
                }
            } else {
                for (int i = 0; i < RW; i++) d = fmaf(qs[i], ld_cache<F32>(cache, base + i), d);
            }
            s = d * scale;
        }
        float cm = vmx_wave_max(s);
        if (lane == 0) red[wave] = cm;
        __syncthreads();
        cm = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
        const float m_new = fmaxf(m, cm);
        const float p = valid ? expf(s - m_new) : 0.f;
        ps[tid] = p;
        float cs = vmx_wave_sum(p);
        if (lane == 0) red[4 + wave] = cs;
        __syncthreads();
        cs = (red[4] + red[5]) + (red[6] + red[7]);
        const float alpha = expf(m - m_new);   // m == -FLT_MAX only before the first chunk without a sink: l and acc are 0 then
        l = l * alpha + cs;
        m = m_new;
#pragma unroll
        for (int i = 0; i < MAXD; i++) acc[i] *= alpha;
        const int cn = min(256, n - c0);
        for (int kk = wave; kk < cn; kk += 4) {
            const float pk = ps[kk];
            const int64_t base = (int64_t)ks[kk] * RW;
#pragma unroll
            for (int i = 0; i < MAXD; i++) {
                const int d = lane + 64 * i;
                if (d < R) acc[i] = fmaf(pk, ld_cache<F32>(cache, base + d), acc[i]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < MAXD; i++) {
        const int d = lane + 64 * i;
        if (d < R) part[wave * R + d] = acc[i];
    }
    __syncthreads();
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = tid; d < R; d += 256)
        out[((int64_t)t * H + h) * R + d] = ((part[d] + part[R + d]) + (part[2 * R + d] + part[3 * R + d])) * inv;
}

}  // namespace

extern "C" int vmx_latent_kv_prepare(const float *fused, int64_t ld_fused, int q_offset, int dkv_offset, const uint16_t *latent_norm_w,
                                     float eps, const float *inv_freq, int rot_dims, const int32_t *positions, const int32_t *slots,
                                     void *cache, int cache_dtype, float *q_rot, int tokens, int heads, int dim, int rot_dim, int kv_rank,
                                     void *stream) {
    VMX_REQUIRE(fused && latent_norm_w && inv_freq && positions && slots && cache && q_rot, "latent_kv_prepare: null pointer");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "latent_kv_prepare: the cache holds f32 or bf16");
    VMX_REQUIRE(heads >= 1 && dim >= 0 && rot_dim >= 0 && kv_rank >= 1, "latent_kv_prepare: bad sizes");
    VMX_REQUIRE(rot_dims >= 0 && rot_dims <= rot_dim && rot_dims % 2 == 0, "latent_kv_prepare: rot_dims (%d) must be even and at most rot_dim (%d)",
                rot_dims, rot_dim);
    if (tokens <= 0) return VMX_OK;
    if (cache_dtype == VMX_F32)
        hipLaunchKernelGGL(latent_prepare_kernel<true>, dim3(tokens), dim3(256), 0, vmx_stream(stream), fused, ld_fused, q_offset, dkv_offset,
                           latent_norm_w, eps, inv_freq, rot_dims, positions, slots, cache, q_rot, heads, dim, rot_dim, kv_rank);
    else
        hipLaunchKernelGGL(latent_prepare_kernel<false>, dim3(tokens), dim3(256), 0, vmx_stream(stream), fused, ld_fused, q_offset, dkv_offset,
                           latent_norm_w, eps, inv_freq, rot_dims, positions, slots, cache, q_rot, heads, dim, rot_dim, kv_rank);
    VMX_CHECK_LAUNCH("latent_kv_prepare");
    return VMX_OK;
}

extern "C" int vmx_latent_attention(float *out_latent, const float *q_abs, const float *q_rot, const void *cache, int cache_dtype,
                                    const int32_t *block_tables, int max_blocks_per_seq, const int32_t *seq_ids, const int32_t *positions,
                                    const uint16_t *sink_bf16, float scale, int window, int tokens, int heads, int kv_rank, int rot_dim,
                                    int block_size, void *stream) {
    VMX_REQUIRE(out_latent && q_abs && q_rot && cache && block_tables && seq_ids && positions, "latent_attention: null pointer");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "latent_attention: the cache holds f32 or bf16");
    VMX_REQUIRE(kv_rank >= 1 && kv_rank <= 512, "latent_attention: kv_rank (%d) must be in 1..512", kv_rank);
    VMX_REQUIRE(heads >= 1 && rot_dim >= 0 && block_size >= 1 && max_blocks_per_seq >= 1 && window >= 0, "latent_attention: bad sizes");
    if (tokens <= 0) return VMX_OK;
    const size_t lds = (size_t)(kv_rank + rot_dim + 256 + 256 + 8 + 4 * kv_rank) * 4;
    dim3 grid(heads, tokens);
    if (cache_dtype == VMX_F32)
        hipLaunchKernelGGL(latent_attn_kernel<true>, grid, dim3(256), lds, vmx_stream(stream), out_latent, q_abs, q_rot, cache, block_tables,
                           max_blocks_per_seq, seq_ids, positions, sink_bf16, scale, window, heads, kv_rank, rot_dim, block_size);
    else
        hipLaunchKernelGGL(latent_attn_kernel<false>, grid, dim3(256), lds, vmx_stream(stream), out_latent, q_abs, q_rot, cache, block_tables,
                           max_blocks_per_seq, seq_ids, positions, sink_bf16, scale, window, heads, kv_rank, rot_dim, block_size);
    VMX_CHECK_LAUNCH("latent_attention");
    return VMX_OK;
}
