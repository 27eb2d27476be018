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

// ---------------------------------------------------------------------------------------------------------------------------
// Matrix-core form (bf16 cache).  A workgroup owns a ROW TILE: 16 (token, head) rows = TPT consecutive tokens x HPT heads, which
// share their keys because the heads of a token read the same cache rows; with 16 or more heads a tile is one token, so decode
// steps fill the matrix instruction as well as prompts do.  Keys are walked in tiles of 64:
//   S = Q K^T     wave w takes keys 16 w .. 16 w + 15 of the tile: Q fragments (the latent-space query | rotated part, rounded to
//                 bf16) stay in registers, key fragments come straight from the cache rows; v_mfma_f32_16x16x32_bf16 leaves lane
//                 (g, n) the scores of rows 4 g .. 4 g + 3 against key n, so a row's maximum and sum are DPP reductions over 16 lanes
//                 plus one exchange between the four waves through LDS;
//   O += P C      the key fragments a wave already holds also go row-major into LDS (one 16-byte write per fragment; the cache is
//                 read once per tile) and come back as C^T through the transposing LDS read (ds_read_b64_tr_b16); wave w owns a
//                 quarter of the latent dimensions of the output; P goes through LDS as a bf16 pair hi + lo (two products), which
//                 keeps the softmax weights at f32 precision.
// A tile whose tokens belong to several sequences (decode steps of models with fewer than 16 heads) is processed once per
// sequence with the other rows masked.  blockIdx.y splits the key range into partitions for launches with few row tiles; their
// (max, sum, O) triples are merged, with the sink, by latent_attn_merge_kernel.
struct LatentAttnArgs {
    float *out;
    const float *q_abs, *q_rot;
    const uint16_t *cache;
    const int32_t *block_tables, *seq_ids, *positions;
    const uint16_t *sink;
    float *part_m, *part_l, *part_o;   // [T][H][NP], [T][H][NP], [T][H][NP][R]
    float scale;
    int max_blocks, window, T, H, R, rd, block_size, HPT, TPT, NHG, NP;
};

constexpr int LA_KT = 64, LA_LD = LA_KT + 8;   // keys per tile; row stride of the P tiles
constexpr int LA_PAD = 32;                    // the row-major latent tile pads its rows by 64 bytes: four consecutive rows, four bank groups
typedef short la_s16x4 __attribute__((ext_vector_type(4)));
typedef short la_s16x8 __attribute__((ext_vector_type(8)));

template <int KSMAX, int DTW>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(const LatentAttnArgs a) {
    extern __shared__ __align__(16) unsigned char la_smem[];
    const int R = a.R, RW = a.R + a.rd;
    const int ROWE = R + LA_PAD;
    uint16_t *KT = reinterpret_cast<uint16_t *>(la_smem);            // [LA_KT][R + LA_PAD]: the tile's latents, row-major
    uint16_t *Phi = KT + (size_t)LA_KT * ROWE;                        // [16][LA_LD]
    uint16_t *Plo = Phi + 16 * LA_LD;                                 // [16][LA_LD]
    float *red_max = reinterpret_cast<float *>(Plo + 16 * LA_LD);     // [4][16]
    float *red_sum = red_max + 64;                                    // [4][16]
    int32_t *sl = reinterpret_cast<int32_t *>(red_sum + 64);          // [64]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, fl = lane & 15, fg = lane >> 4;
    const int tb = blockIdx.x / a.NHG, hg = blockIdx.x % a.NHG, part = blockIdx.y;
    const int t0 = tb * a.TPT, t_end = min(t0 + a.TPT, a.T);
    const int ksteps = (RW + 31) >> 5;
    const int dtiles = (R + 15) >> 4, dt_per_wave = (dtiles + 3) >> 2, dt0 = wave * dt_per_wave;
    for (int first = t0; first < t_end;) {
        const int seq = a.seq_ids[first];
        int last = first;
        while (last + 1 < t_end && a.seq_ids[last + 1] == seq) last++;
        const int32_t *bt = a.block_tables + (int64_t)seq * a.max_blocks;
        const int hi = a.positions[last];
        const int lo = a.window > 0 ? max(0, a.positions[first] - a.window + 1) : 0;
        const int ntiles = (hi - lo) / LA_KT + 1, tpp = (ntiles + a.NP - 1) / a.NP;
        const int kt_begin = part * tpp, kt_end = min(ntiles, kt_begin + tpp);
        // A operand of S: the query of row fl
        uint4 qf[KSMAX];
        {
            const int tq = t0 + fl / a.HPT, hq = hg * a.HPT + fl % a.HPT;
            const bool act = fl < a.TPT * a.HPT && tq >= first && tq <= last && hq < a.H;
#pragma unroll
            for (int s = 0; s < KSMAX; s++) {
                const int k = 32 * s + 8 * fg;
                uint4 v = make_uint4(0, 0, 0, 0);
                if (s < ksteps && act && k < RW) {
                    const float *src = k < R ? a.q_abs + ((int64_t)tq * a.H + hq) * R + k : a.q_rot + ((int64_t)tq * a.H + hq) * a.rd + (k - R);
                    const float4 f0 = *reinterpret_cast<const float4 *>(src), f1 = *reinterpret_cast<const float4 *>(src + 4);
                    const float f[8] = {f0.x, f0.y, f0.z, f0.w, f1.x, f1.y, f1.z, f1.w};
                    v = vmx_pack16x8<false>(f);
                }
                qf[s] = v;
            }
        }
        // the rows this lane holds in accumulator layout: 4 fg + r
        int rpos[4], rlo[4], rtok[4], rhead[4];
        bool ract[4];
        float m_r[4], l_r[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = 4 * fg + r;
            rtok[r] = t0 + row / a.HPT;
            rhead[r] = hg * a.HPT + row % a.HPT;
            ract[r] = row < a.TPT * a.HPT && rtok[r] >= first && rtok[r] <= last && rhead[r] < a.H;
            rpos[r] = ract[r] ? a.positions[rtok[r]] : -1;
            rlo[r] = a.window > 0 ? max(0, rpos[r] - a.window + 1) : 0;
            m_r[r] = -FLT_MAX;
            l_r[r] = 0.f;
        }
        vmx_f32x4 acc[DTW];
#pragma unroll
        for (int d = 0; d < DTW; d++) acc[d] = vmx_f32x4{0.f, 0.f, 0.f, 0.f};
        // cache rows of a tile's keys: looked up one tile ahead, so the block table's latency is not on the tile's critical path
        auto key_slot = [&](int kt) {
            const int j = lo + LA_KT * kt + tid;
            return (tid < LA_KT && kt < kt_end && j <= hi) ? bt[j / a.block_size] * a.block_size + j % a.block_size : -1;
        };
        int next_slot = key_slot(kt_begin);
        for (int kt = kt_begin; kt < kt_end; kt++) {
            const int kbase = lo + LA_KT * kt;
            __syncthreads();   // the previous tile's latents / P / slots have been read
            if (tid < LA_KT) sl[tid] = next_slot;
            __syncthreads();
            next_slot = key_slot(kt + 1);
            // this wave's 16 keys: lane (n, g) reads the 16-byte chunks 32 s + 8 g of key n's cache row.  They are the B operand of
            // the score product and, for the latent part of the row, the tile of the value product: each chunk is also written to
            // KT[key][latent dim], so the cache is read once per tile.
            vmx_f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
            {
                const int slot = sl[16 * wave + fl];
                uint4 kf[KSMAX];
#pragma unroll
                for (int s = 0; s < KSMAX; s++) {
                    const int k = 32 * s + 8 * fg;
                    kf[s] = make_uint4(0, 0, 0, 0);
                    if (s < ksteps && slot >= 0 && k < RW) kf[s] = *reinterpret_cast<const uint4 *>(a.cache + (int64_t)slot * RW + k);
                }
#pragma unroll
                for (int s = 0; s < KSMAX; s++) {
                    const int k = 32 * s + 8 * fg;
                    if (s < ksteps && k < R) *reinterpret_cast<uint4 *>(KT + (16 * wave + fl) * ROWE + k) = kf[s];
                }
#pragma unroll
                for (int s = 0; s < KSMAX; s++)
                    if (s < ksteps)
                        sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, qf[s]), __builtin_bit_cast(vmx_bf16x8, kf[s]), sacc,
                                                                       0, 0, 0);
            }
            const int j = kbase + 16 * wave + fl;
            bool ok[4];
            float sc[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                ok[r] = ract[r] && j <= rpos[r] && j >= rlo[r];
                sc[r] = ok[r] ? sacc[r] * a.scale : -FLT_MAX;
                const float mx = vmx_row16_max(sc[r]);
                if (fl == 0) red_max[wave * 16 + 4 * fg + r] = mx;
            }
            __syncthreads();   // maxima and the transposed latents are in LDS
            float alpha[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = 4 * fg + r;
                const float tm = fmaxf(fmaxf(red_max[row], red_max[16 + row]), fmaxf(red_max[32 + row], red_max[48 + row]));
                const float m_new = fmaxf(m_r[r], tm);
                const float p = ok[r] ? expf(sc[r] - m_new) : 0.f;
                const uint16_t ph = vmx_f32_to_bf16(p);
                Phi[row * LA_LD + 16 * wave + fl] = ph;
                Plo[row * LA_LD + 16 * wave + fl] = vmx_f32_to_bf16(p - vmx_bf16_to_f32(ph));
                const float sm = vmx_row16_sum(p);
                if (fl == 0) red_sum[wave * 16 + row] = sm;
                alpha[r] = expf(m_r[r] - m_new);   // both -FLT_MAX (nothing seen yet): 1, and l and acc are still 0
                m_r[r] = m_new;
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int row = 4 * fg + r;
                l_r[r] = l_r[r] * alpha[r] + ((red_sum[row] + red_sum[16 + row]) + (red_sum[32 + row] + red_sum[48 + row]));
            }
#pragma unroll
            for (int d = 0; d < DTW; d++)
#pragma unroll
                for (int r = 0; r < 4; r++) acc[d][r] *= alpha[r];
#pragma unroll
            for (int ks = 0; ks < LA_KT / 32; ks++) {
                const uint4 ah = *reinterpret_cast<const uint4 *>(Phi + fl * LA_LD + 32 * ks + 8 * fg);
                const uint4 al = *reinterpret_cast<const uint4 *>(Plo + fl * LA_LD + 32 * ks + 8 * fg);
#pragma unroll
                for (int d = 0; d < DTW; d++) {
                    if (d < dt_per_wave && dt0 + d < dtiles) {
                        // B operand = C^T: the transposing LDS read hands lane n the values of column 16 dt + n for the four rows
                        // (keys) its 16-lane group addressed; two reads give the eight keys 32 ks + 8 g .. + 7 of this lane's k slots
                        const uint16_t *src = KT + (32 * ks + 8 * fg + (fl >> 2)) * ROWE + 16 * (dt0 + d) + 4 * (fl & 3);
                        const la_s16x4 c0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((la_s16x4 __attribute__((address_space(3))) *)src);
                        const la_s16x4 c1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((la_s16x4 __attribute__((address_space(3))) *)(src + 4 * ROWE));
                        const la_s16x8 cf = {c0[0], c0[1], c0[2], c0[3], c1[0], c1[1], c1[2], c1[3]};
                        acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, ah), __builtin_bit_cast(vmx_bf16x8, cf), acc[d], 0, 0,
                                                                         0);
                        acc[d] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(vmx_bf16x8, al), __builtin_bit_cast(vmx_bf16x8, cf), acc[d], 0, 0,
                                                                         0);
                    }
                }
            }
        }
        // results of rows 4 fg + r, latent dimensions 16 (dt0 + d) + fl
#pragma unroll
        for (int r = 0; r < 4; r++) {
            if (!ract[r]) continue;
            const int64_t th = (int64_t)rtok[r] * a.H + rhead[r];
            if (a.NP == 1) {
                const float sk = a.sink ? vmx_bf16_to_f32(a.sink[rhead[r]]) : -FLT_MAX;
                const float M = fmaxf(m_r[r], sk), w = expf(m_r[r] - M);
                const float den = l_r[r] * w + (a.sink ? expf(sk - M) : 0.f);
                const float f = den > 0.f ? w / den : 0.f;
#pragma unroll
                for (int d = 0; d < DTW; d++) {
                    const int dim = 16 * (dt0 + d) + fl;
                    if (d < dt_per_wave && dim < R) a.out[th * R + dim] = acc[d][r] * f;
                }
            } else {
                const int64_t tp = th * a.NP + part;
                if (wave == 0 && fl == 0) {
                    a.part_m[tp] = m_r[r];
                    a.part_l[tp] = l_r[r];
                }
#pragma unroll
                for (int d = 0; d < DTW; d++) {
                    const int dim = 16 * (dt0 + d) + fl;
                    if (d < dt_per_wave && dim < R) a.part_o[tp * R + dim] = acc[d][r];
                }
            }
        }
        first = last + 1;
    }
}

// out[t, h] = sum_p e^(m_p - M) O_p / (sum_p e^(m_p - M) l_p + e^(sink - M)), M = max(sink, max_p m_p); NP <= 64.
// Wave 0 turns the partitions' (m, l) into one weight each (one round trip to memory), then every thread sums its dimensions.
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(float *__restrict__ out, const float *__restrict__ part_m,
                                                                 const float *__restrict__ part_l, const float *__restrict__ part_o,
                                                                 const uint16_t *__restrict__ sink, int H, int R, int NP) {
    __shared__ float wgt[64];
    const int64_t th = blockIdx.x;
    if (threadIdx.x < 64) {
        const int p = threadIdx.x;
        const float sk = sink ? vmx_bf16_to_f32(sink[th % H]) : -FLT_MAX;
        const float m = p < NP ? part_m[th * NP + p] : -FLT_MAX, l = p < NP ? part_l[th * NP + p] : 0.f;
        const float M = vmx_wave_max(fmaxf(l > 0.f ? m : -FLT_MAX, sk));
        const float e = l > 0.f ? expf(m - M) : 0.f;
        const float den = vmx_wave_sum(e * l) + (sink ? expf(sk - M) : 0.f);
        wgt[p] = den > 0.f ? e / den : 0.f;
    }
    __syncthreads();
    for (int d = threadIdx.x; d < R; d += 256) {
        float v = 0.f;
        for (int p = 0; p < NP; p++) v = fmaf(wgt[p], part_o[(th * NP + p) * R + d], v);
        out[th * R + d] = v;
    }
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

// Partition count of the matrix-core form for a launch (host arithmetic only): one workgroup fits a compute unit at the largest
// latent size, so the launch is given at most one workgroup per compute unit -- row tiles x partitions <= compute units -- and a
// launch with that many row tiles or more is not split at all.
static int latent_attn_partitions(int tokens, int heads, int window, int max_blocks_per_seq, int block_size) {
    const int hpt = heads < 16 ? heads : 16, tpt = 16 / hpt, nhg = (heads + hpt - 1) / hpt;
    const int64_t tiles = (int64_t)((tokens + tpt - 1) / tpt) * nhg;
    int64_t max_keys = (int64_t)max_blocks_per_seq * block_size;
    if (window > 0 && window < max_keys) max_keys = window;
    const int64_t key_tiles = max_keys / LA_KT + 1;
    int64_t np = vmx_num_cus() / tiles;
    if (np > key_tiles) np = key_tiles;
    if (np > 64) np = 64;
    return np < 1 ? 1 : (int)np;
}

extern "C" size_t vmx_latent_attention_workspace_bytes(int tokens, int heads, int kv_rank, int window, int max_blocks_per_seq,
                                                       int block_size) {
    if (tokens <= 0 || heads <= 0 || kv_rank <= 0 || max_blocks_per_seq <= 0 || block_size <= 0) return 0;
    const int np = latent_attn_partitions(tokens, heads, window, max_blocks_per_seq, block_size);
    return np == 1 ? 0 : (size_t)tokens * heads * np * (kv_rank + 2) * sizeof(float);
}

extern "C" int vmx_latent_attention(float *out_latent, const float *q_abs, const float *q_rot, const void *cache, int cache_dtype,
                                    const int32_t *block_tables, int max_blocks_per_seq, const int32_t *seq_ids, const int32_t *positions,
                                    const uint16_t *sink_bf16, float scale, int window, int tokens, int heads, int kv_rank, int rot_dim,
                                    int block_size, void *workspace, size_t workspace_bytes, void *stream) {
    VMX_REQUIRE(out_latent && q_abs && q_rot && cache && block_tables && seq_ids && positions, "latent_attention: null pointer");
    VMX_REQUIRE(cache_dtype == VMX_F32 || cache_dtype == VMX_BF16, "latent_attention: the cache holds f32 or bf16");
    VMX_REQUIRE(kv_rank >= 1 && kv_rank <= 512, "latent_attention: kv_rank (%d) must be in 1..512", kv_rank);
    VMX_REQUIRE(heads >= 1 && rot_dim >= 0 && block_size >= 1 && max_blocks_per_seq >= 1 && window >= 0, "latent_attention: bad sizes");
    if (tokens <= 0) return VMX_OK;
    hipStream_t st = vmx_stream(stream);
    const int RW = kv_rank + rot_dim;
    // matrix-core form: bf16 cache, 16-byte chunks of a row must not straddle the latent / rotated boundary
    if (cache_dtype == VMX_BF16 && kv_rank % 8 == 0 && rot_dim % 8 == 0 && RW <= 576) {
        LatentAttnArgs a;
        a.out = out_latent, a.q_abs = q_abs, a.q_rot = q_rot, a.cache = (const uint16_t *)cache;
        a.block_tables = block_tables, a.seq_ids = seq_ids, a.positions = positions, a.sink = sink_bf16;
        a.scale = scale, a.max_blocks = max_blocks_per_seq, a.window = window, a.T = tokens, a.H = heads, a.R = kv_rank, a.rd = rot_dim;
        a.block_size = block_size;
        a.HPT = heads < 16 ? heads : 16, a.TPT = 16 / a.HPT, a.NHG = (heads + a.HPT - 1) / a.HPT;
        a.NP = latent_attn_partitions(tokens, heads, window, max_blocks_per_seq, block_size);
        const size_t need = a.NP == 1 ? 0 : (size_t)tokens * heads * a.NP * (kv_rank + 2) * sizeof(float);
        if (need > workspace_bytes || (need && !workspace)) a.NP = 1;   // no room for partitions: one workgroup walks all keys
        a.part_m = (float *)workspace;
        a.part_l = a.part_m + (size_t)tokens * heads * a.NP;
        a.part_o = a.part_l + (size_t)tokens * heads * a.NP;
        const size_t lds = ((size_t)LA_KT * (kv_rank + LA_PAD) + 2 * 16 * LA_LD) * 2 + (64 + 64) * 4 + 64 * 4;
        dim3 grid((unsigned)(((tokens + a.TPT - 1) / a.TPT) * a.NHG), a.NP);
        const bool small = RW <= 160 && kv_rank <= 128;
        const void *fn = small ? (const void *)latent_attn_mfma_kernel<5, 2> : (const void *)latent_attn_mfma_kernel<18, 8>;
        if (lds > 64 * 1024) VMX_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        if (small) hipLaunchKernelGGL((latent_attn_mfma_kernel<5, 2>), grid, dim3(256), lds, st, a);
        else hipLaunchKernelGGL((latent_attn_mfma_kernel<18, 8>), grid, dim3(256), lds, st, a);
        VMX_CHECK_LAUNCH("latent_attention (matrix cores)");
        if (a.NP > 1) {
            hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(tokens * heads), dim3(256), 0, st, out_latent, a.part_m, a.part_l, a.part_o, sink_bf16,
                               heads, kv_rank, a.NP);
            VMX_CHECK_LAUNCH("latent_attention (merge)");
        }
        return VMX_OK;
    }
    const size_t lds = (size_t)(kv_rank + rot_dim + 256 + 256 + 8 + 4 * kv_rank) * 4;
    dim3 grid(heads, tokens);
    if (cache_dtype == VMX_F32)
        hipLaunchKernelGGL(latent_attn_kernel<true>, grid, dim3(256), lds, st, out_latent, q_abs, q_rot, cache, block_tables,
                           max_blocks_per_seq, seq_ids, positions, sink_bf16, scale, window, heads, kv_rank, rot_dim, block_size);
    else
        hipLaunchKernelGGL(latent_attn_kernel<false>, grid, dim3(256), lds, st, out_latent, q_abs, q_rot, cache, block_tables,
                           max_blocks_per_seq, seq_ids, positions, sink_bf16, scale, window, heads, kv_rank, rot_dim, block_size);
    VMX_CHECK_LAUNCH("latent_attention");
    return VMX_OK;
}
