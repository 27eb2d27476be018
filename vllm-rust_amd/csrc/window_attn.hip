// Grouped-query attention over a paged key/value cache for packed steps, with the score shaping some decoder families use:
//   s_j = (q . k_j) * scale * temp[h];  s_j <- cap * tanh(s_j / cap) (cap > 0);  p = softmax over the visible j;  o = sum_j p_j v_j
// Position i of a sequence sees j <= i when i - j < window (window 0: every earlier key) or j < keep_first (the first tokens of
// the sequence stay visible after the window has passed them).  No rotation: positions only decide visibility.  Query head h
// reads key/value head h / (heads / kv_heads); key and value widths may differ.  The head's output may be multiplied by
// sigmoid(gate[t, h]) (one number per token and head) before it is stored.
//
// Keys and values live in two caches of rows [kv_heads * dim] / [kv_heads * vdim], bf16 or f32; a step writes its new rows first
// (vmx_kv_cache_write_f32) and prompts, prompt portions and decode tokens then run the SAME kernel over the cache, so a row's
// result does not depend on how its prompt was cut or on what else is in the step.  Scores, softmax and the weighted sum are f32.
// The visible keys of a row are two runs, [0, min(keep_first, lo)) and [lo, i] with lo = max(0, i - window + 1); a wave owns one
// (token, head) row and walks them 64 at a time: lane l scores key l of the tile, then every lane sums its value columns.
#include "vmx_kernels.h"
#include <float.h>

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
};

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
    float g = 1.0f / den;
    if (p.gate) g *= 1.0f / (1.0f + expf(-p.gate[(int64_t)t * p.ldgate + h]));
#pragma unroll
    for (int u = 0; u < VPL; u++) {
        const int c = lane + 64 * u;
        if (c < V) {
            const int64_t o = ((int64_t)t * p.heads + h) * V + c;
            if (p.out_f32) ((float *)p.out)[o] = acc[u] * g;
            else ((uint16_t *)p.out)[o] = vmx_f32_to_bf16(acc[u] * g);
        }
    }
}

}  // namespace

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

extern "C" int vmx_window_attention(void *out, int out_dtype, const float *q, int64_t ldq, const void *k_cache, const void *v_cache,
                                    int cache_dtype, const int32_t *block_tables, int max_blocks_per_seq, const int32_t *seq_ids,
                                    const int32_t *positions, const uint16_t *head_temp_bf16, const float *gate, int64_t ldgate, float scale,
                                    float softcap, int window, int keep_first, int tokens, int heads, int kv_heads, int dim, int vdim,
                                    int block_size, void *stream) {
    VMX_REQUIRE(out && q && k_cache && v_cache && block_tables && seq_ids && positions, "window_attention: null pointer");
    VMX_REQUIRE((out_dtype == VMX_F32 || out_dtype == VMX_BF16) && (cache_dtype == VMX_F32 || cache_dtype == VMX_BF16),
                "window_attention: f32 or bf16 output and cache");
    VMX_REQUIRE(heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0, "window_attention: %d query heads do not share %d key/value heads evenly",
                heads, kv_heads);
    VMX_REQUIRE(dim >= 1 && dim <= WA_MAX_DIM && vdim >= 1 && vdim <= 256, "window_attention: head sizes %d / %d outside 1..256", dim, vdim);
    VMX_REQUIRE(window >= 0 && keep_first >= 0 && block_size >= 1 && max_blocks_per_seq >= 1 && softcap >= 0.f, "window_attention: bad arguments");
    VMX_REQUIRE(ldq >= (int64_t)heads * dim && (!gate || ldgate >= heads), "window_attention: bad row strides");
    if (tokens <= 0) return VMX_OK;
    WinAttn p{out, out_dtype == VMX_F32, q, ldq, k_cache, v_cache, block_tables, seq_ids, positions, max_blocks_per_seq, head_temp_bf16,
              gate, ldgate, scale, softcap, window, keep_first, tokens, heads, kv_heads, dim, vdim, block_size};
    const dim3 grid((tokens * heads + 3) / 4), block(256);
    hipStream_t st = vmx_stream(stream);
    const bool f32 = cache_dtype == VMX_F32;
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
