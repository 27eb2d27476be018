// Whole-step executor of the Gesutar decoder family: a stack of pre-norm layers, each a token mixer plus an optional
// feed-forward, described layer by layer in the model's configuration (sizes, windows and constants may differ between layers).
//   x = embed[token] * scale + bigram[(prev * mul_prev + token * mul_cur) mod buckets]      (row `buckets` for a first token)
//   x += mixer(rms_norm(x, norm1));  x += ff(rms_norm(x, norm2));  logits = head . rms_norm(x, final.norm)
// Mixer "latent_attention" (latent_attn.hip): low-rank compressed keys/values in a paged cache, sliding window, per-head sink,
// sigmoid output gate.  Feed-forward "moe": softmax router with group-limited top-k (moe_kernels.hip), squared-ReLU experts run
// as token-grouped products over pairs sorted by expert, plus an always-on shared expert.
//
// One entry point serves prompts, prompt portions and decode steps: the step's tokens are PACKED ([tokens] arrays of token id,
// previous token id, position, cache slot and sequence index; [sequences, max_blocks] block tables), so requests of unequal
// length need no padding and a row's arithmetic never depends on what else is in the step.  The residual stream, norms, the
// router, rotations, scores and softmax are f32 in both modes; in VMX_BF16 mode the linears take bf16 operands (f32
// accumulation) and the cache holds bf16, in VMX_F32 mode every product is a true f32 product and the cache holds f32.
// Like the other executors the forward call allocates nothing, reads nothing back and is graph-capturable.
#include "vmx_kernels.h"
#include <float.h>
#include <math.h>
#include <string>
#include <vector>

namespace {

using Buf = VmxBuf;

struct Layer {
    vmx_gesutar_layer_config c;
    Buf norm1, norm2, wfused, dkv_norm, uk, uk_t, uv, sink, wo, router, eup, edown, sup, sdown, inv_freq, cache;
    int q_off = 0, dkv_off = 0, g_off = 0, nf = 0;
    std::vector<std::string> missing;   // tensor names not loaded yet
};

}  // namespace

struct vmx_gesutar {
    vmx_gesutar_config cfg;
    std::vector<Layer> layers;
    Buf embed, bigram, final_norm, head;
    std::vector<std::string> missing;
    // step workspaces, sized for max_tokens
    Buf x, h, fused, qabs, qrot, olat, attn, attn_ws, argmax_keys, few_pairs, rlogits, topw, topi, sorted, blk_expert, total, inv, act, ydown, sact, sout, hsel;
    int sorted_cap = 0;
    bool f32() const { return cfg.dtype == VMX_F32; }
    size_t esz() const { return f32() ? 4 : 2; }
};

namespace {

// x[t] = embed[token] * scale + bigram[row]
__global__ __launch_bounds__(256) void embed_bigram_kernel(float *__restrict__ x, const uint16_t *__restrict__ embed,
                                                            const uint16_t *__restrict__ bigram, const int32_t *__restrict__ tokens,
                                                            const int32_t *__restrict__ prev, int width, int vocab, float scale, int buckets,
                                                            int mul_prev, int mul_cur) {
    const int t = blockIdx.x;
    int id = tokens[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int pv = prev[t];
    int64_t row = buckets;
    if (pv >= 0) row = ((int64_t)pv * mul_prev + (int64_t)id * mul_cur) % buckets;
    for (int i = threadIdx.x; i < width; i += 256) {
        float v = vmx_bf16_to_f32(embed[(int64_t)id * width + i]) * scale;
        if (buckets > 0) v += vmx_bf16_to_f32(bigram[row * width + i]);
        x[(int64_t)t * width + i] = v;
    }
}

// out[h][r][d] = in[h][d][r]: the key up-projection as [head][latent][dim], so that qa_h = U_h^T q_h reads its weights along k
__global__ __launch_bounds__(256) void transpose_heads_kernel(uint16_t *__restrict__ out, const uint16_t *__restrict__ in, int H, int D, int R) {
    const int64_t n = (int64_t)H * D * R;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
        const int64_t h = i / ((int64_t)D * R), rem = i % ((int64_t)D * R);
        const int r = (int)(rem / D), d = (int)(rem % D);
        out[i] = in[(h * D + d) * R + r];
    }
}

int upload(Buf &b, size_t offset, const void *data, size_t bytes, hipStream_t st) {
    VMX_CHECK_HIP(hipMemcpyAsync((char *)b.p + offset, data, bytes, hipMemcpyDefault, st));
    VMX_CHECK_HIP(hipStreamSynchronize(st));
    return VMX_OK;
}

void erase_name(std::vector<std::string> &v, const std::string &n) {
    for (size_t i = 0; i < v.size(); i++)
        if (v[i] == n) {
            v.erase(v.begin() + i);
            return;
        }
}

}  // namespace

extern "C" int vmx_gesutar_create(const vmx_gesutar_config *cfg, const vmx_gesutar_layer_config *layer_cfgs, vmx_gesutar **out) {
    VMX_REQUIRE(cfg && layer_cfgs && out, "gesutar_create: null pointer");
    const vmx_gesutar_config &c = *cfg;
    VMX_REQUIRE(c.vocab >= 1 && c.width >= 1 && c.num_layers >= 1, "gesutar_create: bad sizes (vocab %d, width %d, layers %d)", c.vocab, c.width,
                c.num_layers);
    VMX_REQUIRE(c.dtype == VMX_F32 || c.dtype == VMX_BF16, "gesutar_create: dtype must be VMX_F32 or VMX_BF16");
    VMX_REQUIRE(c.block_size >= 1 && c.num_blocks >= 1 && c.max_tokens >= 1 && c.max_seqs >= 1, "gesutar_create: bad cache / batch geometry");
    VMX_REQUIRE(c.bigram_buckets >= 0, "gesutar_create: bigram buckets must not be negative");
    vmx_gesutar *m = new vmx_gesutar();
    m->cfg = c;
    m->layers.resize(c.num_layers);
    const size_t T = c.max_tokens, W = c.width;
    size_t maxr = 0, nf = 0, hr = 0, hrd = 0, hv = 0, ne = 1, pairs = 0, eff = 0, sff = 0, cap = 0;
    int rc = VMX_OK;
#define GA(buf, n)                       \
    do {                                 \
        if (!rc) rc = (buf).alloc(n);    \
    } while (0)
    for (int li = 0; li < c.num_layers && !rc; li++) {
        Layer &L = m->layers[li];
        L.c = layer_cfgs[li];
        const vmx_gesutar_layer_config &lc = L.c;
        const std::string pre = "l" + std::to_string(li) + ".";
        if (lc.mixer != VMX_MIXER_LATENT_ATTENTION) {
            vmx_set_error("gesutar_create: layer %d: unknown mixer kind %d", li, lc.mixer);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        if (lc.heads < 1 || lc.dim < 0 || lc.rot_dim < 0 || lc.dim + lc.rot_dim < 1 || lc.vdim < 1 || lc.kv_rank < 1 || lc.kv_rank > 512 ||
            lc.window < 0 || lc.rot_dims < 0 || lc.rot_dims > lc.rot_dim || lc.rot_dims % 2) {
            vmx_set_error("gesutar_create: layer %d: bad latent-attention sizes", li);
            rc = VMX_EINVAL;
            break;
        }
        const size_t nq = (size_t)lc.heads * (lc.dim + lc.rot_dim), ng = (size_t)lc.heads * lc.vdim, nkv = (size_t)lc.kv_rank + lc.rot_dim;
        L.q_off = 0;
        L.dkv_off = (int)nq;
        L.g_off = (int)(nq + nkv);
        L.nf = (int)(nq + nkv + ng);
        GA(L.norm1, W * 2);
        GA(L.wfused, (size_t)L.nf * W * 2);
        GA(L.dkv_norm, (size_t)lc.kv_rank * 2);
        GA(L.uk, (size_t)lc.heads * lc.dim * lc.kv_rank * 2);
        GA(L.uk_t, (size_t)lc.heads * lc.dim * lc.kv_rank * 2);
        GA(L.uv, (size_t)lc.heads * lc.vdim * lc.kv_rank * 2);
        GA(L.sink, (size_t)lc.heads * 2);
        GA(L.wo, W * ng * 2);
        GA(L.cache, (size_t)c.num_blocks * c.block_size * nkv * m->esz());
        GA(L.inv_freq, (size_t)(lc.rot_dims / 2 + 1) * 4);
        if (!rc) {
            std::vector<float> f(lc.rot_dims / 2 + 1, 0.f);
            for (int i = 0; i < lc.rot_dims / 2; i++) f[i] = (float)pow(lc.rot_base, -2.0 * i / (double)lc.rot_dims);
            if (hipMemcpy(L.inv_freq.p, f.data(), f.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
                vmx_set_error("gesutar_create: upload failed");
                rc = VMX_ELAUNCH;
            }
        }
        for (const char *n : {"norm1", "mix.q", "mix.dkv", "mix.dkv.norm", "mix.uk", "mix.uv", "mix.sink", "mix.g", "mix.o"}) L.missing.push_back(pre + n);
        if (lc.mlp == VMX_MLP_MOE) {
            if (lc.experts < 1 || lc.experts > 256 || lc.top < 1 || lc.groups < 1 || lc.experts % lc.groups || lc.keep_groups < 1 ||
                lc.keep_groups > lc.groups || lc.top > lc.keep_groups * (lc.experts / lc.groups) || lc.expert_ff < 1 || lc.shared_ff < 0) {
                vmx_set_error("gesutar_create: layer %d: bad mixture-of-experts sizes", li);
                rc = VMX_EINVAL;
                break;
            }
            GA(L.norm2, W * 2);
            GA(L.router, (size_t)lc.experts * W * 2);
            GA(L.eup, (size_t)lc.experts * lc.expert_ff * W * 2);
            GA(L.edown, (size_t)lc.experts * lc.expert_ff * W * 2);
            L.missing.push_back(pre + "norm2");
            L.missing.push_back(pre + "mlp.router");
            for (int e = 0; e < lc.experts; e++) {
                L.missing.push_back(pre + "mlp.e" + std::to_string(e) + ".up");
                L.missing.push_back(pre + "mlp.e" + std::to_string(e) + ".down");
            }
            if (lc.shared_ff > 0) {
                GA(L.sup, (size_t)lc.shared_ff * W * 2);
                GA(L.sdown, (size_t)lc.shared_ff * W * 2);
                L.missing.push_back(pre + "mlp.shared.up");
                L.missing.push_back(pre + "mlp.shared.down");
            }
            ne = std::max(ne, (size_t)lc.experts);
            pairs = std::max(pairs, T * lc.top);
            cap = std::max(cap, std::max(T * lc.top + (size_t)lc.experts * 63, (size_t)VMX_MOE_FEW_PAIRS * 16));
            eff = std::max(eff, (size_t)lc.expert_ff);
            sff = std::max(sff, (size_t)lc.shared_ff);
        } else if (lc.mlp != VMX_MLP_NONE) {
            vmx_set_error("gesutar_create: layer %d: unknown feed-forward kind %d", li, lc.mlp);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        nf = std::max(nf, (size_t)L.nf);
        maxr = std::max(maxr, (size_t)lc.kv_rank);
        hr = std::max(hr, (size_t)lc.heads * lc.kv_rank);
        hrd = std::max(hrd, (size_t)lc.heads * lc.rot_dim);
        hv = std::max(hv, ng);
    }
    GA(m->embed, (size_t)c.vocab * W * 2);
    GA(m->bigram, (size_t)(c.bigram_buckets + 1) * W * 2);
    GA(m->final_norm, W * 2);
    GA(m->head, (size_t)c.vocab * W * 2);
    m->missing = {"embed", "final.norm", "head"};
    if (c.bigram_buckets > 0) m->missing.push_back("bigram");
    GA(m->x, T * W * 4);
    GA(m->h, T * W * m->esz());
    GA(m->hsel, T * W * m->esz());
    GA(m->fused, T * nf * 4);
    GA(m->qabs, T * hr * 4);
    GA(m->qrot, T * (hrd + 1) * 4);
    GA(m->olat, T * hr * 4);
    GA(m->attn_ws, (size_t)24576 * (maxr + 2) * 4);   // key partitions of launches with few rows: tokens x heads x partitions < 24576
    GA(m->attn, T * hv * m->esz());
    GA(m->argmax_keys, T * ((size_t)c.vocab / VMX_ARGMAX_CHUNK + 1) * 8);
    GA(m->few_pairs, (size_t)(2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS + 1) * 4);
    GA(m->rlogits, T * ne * 4);
    GA(m->topw, (pairs + 1) * 4);
    GA(m->topi, (pairs + 1) * 4);
    GA(m->sorted, (cap + 1) * 4);
    GA(m->blk_expert, (cap / 16 + 2) * 4);
    GA(m->total, 16);
    GA(m->inv, (pairs + 1) * 4);
    GA(m->act, (cap + 1) * eff * m->esz());
    GA(m->ydown, (cap + 1) * W * 4);
    GA(m->sact, T * (sff + 1) * m->esz());
    GA(m->sout, T * W * 4);
#undef GA
    if (!rc) {
        // decode steps with a handful of (token, slot) pairs skip the sort: pair p is its own 16-row block (row 16 p)
        std::vector<int32_t> fp(2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS + 1);
        for (int i = 0; i < VMX_MOE_FEW_PAIRS * 16; i++) {
            fp[i] = i % 16 == 0 ? i / 16 : 0x7fffffff;                        // gathered rows of the up product: pair index or padding
            fp[VMX_MOE_FEW_PAIRS * 16 + i] = i % 16 == 0 ? i : 0x7fffffff;            // rows of the down product: themselves or padding
        }
        for (int p = 0; p < VMX_MOE_FEW_PAIRS; p++) fp[2 * VMX_MOE_FEW_PAIRS * 16 + p] = 16 * p;   // where pair p's result lies
        fp[2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS] = 0x7fffffff;                       // "total rows": never cuts
        if (hipMemcpy(m->few_pairs.p, fp.data(), fp.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
            vmx_set_error("gesutar_create: upload failed");
            rc = VMX_ELAUNCH;
        }
    }
    m->sorted_cap = (int)cap;
    if (rc) {
        vmx_gesutar_destroy(m);
        return rc;
    }
    *out = m;
    return VMX_OK;
}

extern "C" void vmx_gesutar_destroy(vmx_gesutar *m) {
    if (!m) return;
    for (Layer &L : m->layers)
        for (Buf *b : {&L.norm1, &L.norm2, &L.wfused, &L.dkv_norm, &L.uk, &L.uk_t, &L.uv, &L.sink, &L.wo, &L.router, &L.eup, &L.edown, &L.sup, &L.sdown,
                       &L.inv_freq, &L.cache})
            b->release();
    for (Buf *b : {&m->embed, &m->bigram, &m->final_norm, &m->head, &m->x, &m->h, &m->fused, &m->qabs, &m->qrot, &m->olat, &m->attn, &m->attn_ws, &m->argmax_keys, &m->few_pairs, &m->rlogits,
                   &m->topw, &m->topi, &m->sorted, &m->blk_expert, &m->total, &m->inv, &m->act, &m->ydown, &m->sact, &m->sout, &m->hsel})
        b->release();
    delete m;
}

// One checkpoint tensor by its name in the file (bf16, shape [out, in] for matrices).  `data` may be host or device memory.
extern "C" int vmx_gesutar_load_tensor(vmx_gesutar *m, const char *name, const void *data, size_t bytes, void *stream) {
    VMX_REQUIRE(m && name && (data || bytes == 0), "gesutar_load_tensor: null pointer");
    hipStream_t st = vmx_stream(stream);
    const vmx_gesutar_config &c = m->cfg;
    const size_t W = c.width;
    const std::string n(name);
    Buf *dst = nullptr;
    size_t off = 0, need = 0;
    std::vector<std::string> *missing = &m->missing;
    if (n == "embed") dst = &m->embed, need = (size_t)c.vocab * W * 2;
    else if (n == "bigram" && c.bigram_buckets > 0) dst = &m->bigram, need = (size_t)(c.bigram_buckets + 1) * W * 2;
    else if (n == "final.norm") dst = &m->final_norm, need = W * 2;
    else if (n == "head") dst = &m->head, need = (size_t)c.vocab * W * 2;
    else if (n.size() > 1 && n[0] == 'l' && isdigit((unsigned char)n[1])) {
        size_t dot = n.find('.');
        VMX_REQUIRE(dot != std::string::npos, "gesutar_load_tensor: unknown tensor `%s`", name);
        const int li = atoi(n.substr(1, dot - 1).c_str());
        VMX_REQUIRE(li >= 0 && li < c.num_layers, "gesutar_load_tensor: `%s`: the model has %d layers", name, c.num_layers);
        Layer &L = m->layers[li];
        const vmx_gesutar_layer_config &lc = L.c;
        missing = &L.missing;
        const std::string s = n.substr(dot + 1);
        const size_t nq = (size_t)lc.heads * (lc.dim + lc.rot_dim), ng = (size_t)lc.heads * lc.vdim, nkv = (size_t)lc.kv_rank + lc.rot_dim;
        const bool moe = lc.mlp == VMX_MLP_MOE;
        if (s == "norm1") dst = &L.norm1, need = W * 2;
        else if (s == "norm2" && moe) dst = &L.norm2, need = W * 2;
        else if (s == "mix.q") dst = &L.wfused, off = (size_t)L.q_off * W * 2, need = nq * W * 2;
        else if (s == "mix.dkv") dst = &L.wfused, off = (size_t)L.dkv_off * W * 2, need = nkv * W * 2;
        else if (s == "mix.g") dst = &L.wfused, off = (size_t)L.g_off * W * 2, need = ng * W * 2;
        else if (s == "mix.dkv.norm") dst = &L.dkv_norm, need = (size_t)lc.kv_rank * 2;
        else if (s == "mix.uk") dst = &L.uk, need = (size_t)lc.heads * lc.dim * lc.kv_rank * 2;
        else if (s == "mix.uv") dst = &L.uv, need = (size_t)lc.heads * lc.vdim * lc.kv_rank * 2;
        else if (s == "mix.sink") dst = &L.sink, need = (size_t)lc.heads * 2;
        else if (s == "mix.o") dst = &L.wo, need = W * ng * 2;
        else if (moe && s == "mlp.router") dst = &L.router, need = (size_t)lc.experts * W * 2;
        else if (moe && lc.shared_ff > 0 && s == "mlp.shared.up") dst = &L.sup, need = (size_t)lc.shared_ff * W * 2;
        else if (moe && lc.shared_ff > 0 && s == "mlp.shared.down") dst = &L.sdown, need = (size_t)lc.shared_ff * W * 2;
        else if (moe && s.rfind("mlp.e", 0) == 0) {
            const size_t d2 = s.find('.', 5);
            VMX_REQUIRE(d2 != std::string::npos && d2 > 5, "gesutar_load_tensor: unknown tensor `%s`", name);
            const int e = atoi(s.substr(5, d2 - 5).c_str());
            VMX_REQUIRE(e >= 0 && e < lc.experts, "gesutar_load_tensor: `%s`: the layer has %d experts", name, lc.experts);
            const std::string part = s.substr(d2 + 1);
            need = (size_t)lc.expert_ff * W * 2;
            off = (size_t)e * need;
            if (part == "up") dst = &L.eup;
            else if (part == "down") dst = &L.edown;
        }
    }
    VMX_REQUIRE(dst, "gesutar_load_tensor: unknown tensor `%s`", name);
    VMX_REQUIRE(bytes == need, "gesutar_load_tensor: `%s`: expected %zu bytes of bf16, got %zu", name, need, bytes);
    if (bytes > 0) {
        if (int rc = upload(*dst, off, data, bytes, st)) return rc;
        if (n.size() > 7 && n.compare(n.size() - 7, 7, ".mix.uk") == 0) {
            Layer &L = m->layers[atoi(n.substr(1).c_str())];
            hipLaunchKernelGGL(transpose_heads_kernel, dim3(512), dim3(256), 0, st, L.uk_t.as<uint16_t>(), L.uk.as<uint16_t>(), L.c.heads, L.c.dim,
                               L.c.kv_rank);
            VMX_CHECK_LAUNCH("gesutar transpose");
            VMX_CHECK_HIP(hipStreamSynchronize(st));
        }
    }
    erase_name(*missing, n);
    return VMX_OK;
}

// Number of checkpoint tensors still to load; the error text names the first.
extern "C" int vmx_gesutar_missing_tensors(const vmx_gesutar *m) {
    if (!m) return -1;
    size_t n = m->missing.size();
    const std::string *first = m->missing.empty() ? nullptr : &m->missing[0];
    for (const Layer &L : m->layers) {
        if (!first && !L.missing.empty()) first = &L.missing[0];
        n += L.missing.size();
    }
    if (first) vmx_set_error("gesutar: %zu tensors not loaded, first `%s`", n, first->c_str());
    return (int)n;
}

extern "C" int vmx_gesutar_forward(vmx_gesutar *m, const int32_t *tokens, const int32_t *prev_tokens, const int32_t *positions,
                                   const int32_t *slots, const int32_t *seq_ids, int num_tokens, const int32_t *block_tables, int num_seqs,
                                   int max_blocks_per_seq, const int32_t *logit_rows, int num_logit_rows, float *logits, int32_t *greedy_ids,
                                   float *layer_trace, void *stream) {
    VMX_REQUIRE(m && tokens && prev_tokens && positions && slots && seq_ids && block_tables, "gesutar_forward: null pointer");
    const vmx_gesutar_config &c = m->cfg;
    VMX_REQUIRE(num_tokens >= 1 && num_tokens <= c.max_tokens, "gesutar_forward: %d tokens, the model was created for at most %d", num_tokens,
                c.max_tokens);
    VMX_REQUIRE(num_seqs >= 1 && max_blocks_per_seq >= 1, "gesutar_forward: bad block-table shape");
    VMX_REQUIRE(num_logit_rows >= 0 && num_logit_rows <= num_tokens && (num_logit_rows == 0 || (logit_rows && (logits || greedy_ids))),
                "gesutar_forward: bad logit rows");
    if (vmx_gesutar_missing_tensors(m) != 0) return VMX_EINVAL;   // the message names the first missing tensor
    hipStream_t st = vmx_stream(stream);
    const int T = num_tokens, W = c.width, f32 = m->f32() ? 1 : 0;
    const int cdt = f32 ? VMX_F32 : VMX_BF16;
    float *x = m->x.as<float>();
    hipLaunchKernelGGL(embed_bigram_kernel, dim3(T), dim3(256), 0, st, x, m->embed.as<uint16_t>(), m->bigram.as<uint16_t>(), tokens, prev_tokens,
                       W, c.vocab, (float)c.embed_scale, c.bigram_buckets, c.bigram_mul_prev, c.bigram_mul_cur);
    VMX_CHECK_LAUNCH("gesutar embed");
    for (int li = 0; li < c.num_layers; li++) {
        Layer &L = m->layers[li];
        const vmx_gesutar_layer_config &lc = L.c;
        const int H = lc.heads, R = lc.kv_rank, rd = lc.rot_dim, dim = lc.dim, vd = lc.vdim;
        // ---- mixer: latent attention
        if (int rc = vmx_rms_norm_f32in(m->h.p, f32, x, nullptr, L.norm1.as<uint16_t>(), 0, W, c.norm_eps, T, st)) return rc;
        VmxLinear p;
        p.A = m->h.p, p.a_f32 = f32, p.lda = W;
        p.W = L.wfused.as<uint16_t>(), p.w_sn = W, p.w_sk = 1;
        p.C = m->fused.p, p.c_f32 = 1, p.ldc = L.nf;
        p.M = T, p.N = L.nf, p.K = W, p.exact = f32;
        if (int rc = vmx_linear_launch(p, st)) return rc;   // q | dkv | gate in one product
        if (int rc = vmx_latent_kv_prepare(m->fused.as<float>(), L.nf, L.q_off, L.dkv_off, L.dkv_norm.as<uint16_t>(), c.norm_eps,
                                           L.inv_freq.as<float>(), lc.rot_dims, positions, slots, L.cache.p, cdt, m->qrot.as<float>(), T, H, dim,
                                           rd, R, st))
            return rc;
        if (dim > 0) {   // qa_h = U_h^T q_h: per head, [T, dim] x [dim, R]
            VmxLinear a;
            a.A = m->fused.as<float>() + L.q_off, a.a_f32 = 1, a.lda = L.nf, a.a_bs = dim + rd;
            a.W = L.uk_t.as<uint16_t>(), a.w_sn = dim, a.w_sk = 1, a.w_bs = (int64_t)dim * R;
            a.C = m->qabs.p, a.c_f32 = 1, a.ldc = (int64_t)H * R, a.c_bs = R;
            a.M = T, a.N = R, a.K = dim, a.batch = H, a.exact = f32;
            if (int rc = vmx_linear_launch(a, st)) return rc;
        } else {
            if (int rc = vmx_zero_f32(m->qabs.as<float>(), (int64_t)T * H * R, st)) return rc;
        }
        if (int rc = vmx_latent_attention(m->olat.as<float>(), m->qabs.as<float>(), m->qrot.as<float>(), L.cache.p, cdt, block_tables,
                                          max_blocks_per_seq, seq_ids, positions, L.sink.as<uint16_t>(), lc.scale, lc.window, T, H, R, rd,
                                          c.block_size, m->attn_ws.p, m->attn_ws.bytes, st))
            return rc;
        {   // v_h = V_h o_h, times sigmoid(gate): per head, [T, R] x [vd, R]^T
            VmxLinear v;
            v.A = m->olat.p, v.a_f32 = 1, v.lda = (int64_t)H * R, v.a_bs = R;
            v.W = L.uv.as<uint16_t>(), v.w_sn = R, v.w_sk = 1, v.w_bs = (int64_t)vd * R;
            v.C = m->attn.p, v.c_f32 = f32, v.ldc = (int64_t)H * vd, v.c_bs = vd;
            v.M = T, v.N = vd, v.K = R, v.batch = H, v.exact = f32;
            v.epilogue = VMX_EP_MUL_SIGMOID, v.aux = m->fused.as<float>() + L.g_off, v.ldaux = L.nf, v.aux_bs = vd;
            if (int rc = vmx_linear_launch(v, st)) return rc;
        }
        {   // x += W_o attn
            VmxLinear o;
            o.A = m->attn.p, o.a_f32 = f32, o.lda = (int64_t)H * vd;
            o.W = L.wo.as<uint16_t>(), o.w_sn = (int64_t)H * vd, o.w_sk = 1;
            o.C = x, o.c_f32 = 1, o.ldc = W;
            o.M = T, o.N = W, o.K = H * vd, o.exact = f32, o.epilogue = VMX_EP_ADD_F32;
            if (int rc = vmx_linear_launch(o, st)) return rc;
        }
        // ---- feed-forward: mixture of experts
        if (lc.mlp == VMX_MLP_MOE) {
            const int E = lc.experts, k = lc.top, ff = lc.expert_ff, pairs = T * k;
            if (int rc = vmx_rms_norm_f32in(m->h.p, f32, x, nullptr, L.norm2.as<uint16_t>(), 0, W, c.norm_eps, T, st)) return rc;
            VmxLinear r;   // router logits: always a true f32 product
            r.A = m->h.p, r.a_f32 = f32, r.lda = W;
            r.W = L.router.as<uint16_t>(), r.w_sn = W, r.w_sk = 1;
            r.C = m->rlogits.p, r.c_f32 = 1, r.ldc = E;
            r.M = T, r.N = E, r.K = W, r.exact = 1;
            if (int rc = vmx_linear_launch(r, st)) return rc;
            // logits and routing stay two launches: one workgroup per token doing both walks K once per 16 experts in sequence
            // (21.5 us at one row of 2048 against 10.3 + 5.7 us for the pair)
            if (int rc = vmx_grouped_topk_router(m->rlogits.as<float>(), m->topw.as<float>(), m->topi.as<int32_t>(), T, E, k, lc.groups,
                                                 lc.keep_groups, lc.router_scale, st))
                return rc;
            const bool few = pairs <= VMX_MOE_FEW_PAIRS;   // every pair its own block: no sort, an expert's weights are read once per pair
            const int br = few ? 16 : (pairs >= 32 * E ? 64 : 16);
            const int cap = few ? pairs * 16 : pairs + E * (br - 1);
            const int32_t *fp = m->few_pairs.as<int32_t>();
            const int32_t *up_rows = few ? fp : m->sorted.as<int32_t>(), *down_rows = few ? fp + VMX_MOE_FEW_PAIRS * 16 : nullptr;
            const int32_t *blk = few ? m->topi.as<int32_t>() : m->blk_expert.as<int32_t>();
            const int32_t *total = few ? fp + 2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS : m->total.as<int32_t>();
            const int32_t *inv = few ? fp + 2 * VMX_MOE_FEW_PAIRS * 16 : m->inv.as<int32_t>();
            if (!few) {
                if (int rc = vmx_moe_align_block_size(m->topi.as<int32_t>(), m->sorted.as<int32_t>(), m->blk_expert.as<int32_t>(),
                                                      m->total.as<int32_t>(), pairs, E, br, cap, st))
                    return rc;
                if (int rc = vmx_moe_inverse(m->inv.as<int32_t>(), m->sorted.as<int32_t>(), m->total.as<int32_t>(), pairs, cap, st)) return rc;
            }
            VmxLinear u;   // act = relu(W_up[e] h)^2 over the pairs' rows
            u.A = m->h.p, u.a_f32 = f32, u.lda = W;
            u.W = L.eup.as<uint16_t>(), u.w_sn = W, u.w_sk = 1;
            u.C = m->act.p, u.c_f32 = f32, u.ldc = ff;
            u.M = cap, u.N = ff, u.K = W, u.exact = f32, u.epilogue = VMX_EP_RELU2;
            u.row_ids = up_rows, u.row_div = k, u.row_limit = pairs;
            u.block_expert = blk, u.expert_stride = (int64_t)ff * W, u.block_rows = br, u.total_rows = total;
            if (int rc = vmx_linear_launch(u, st)) return rc;
            VmxLinear d;   // y = W_down[e] act
            d.A = m->act.p, d.a_f32 = f32, d.lda = ff;
            d.W = L.edown.as<uint16_t>(), d.w_sn = ff, d.w_sk = 1;
            d.C = m->ydown.p, d.c_f32 = 1, d.ldc = W;
            d.M = cap, d.N = W, d.K = ff, d.exact = f32;
            d.row_ids = down_rows, d.row_div = 1, d.row_limit = cap;
            d.block_expert = blk, d.expert_stride = (int64_t)ff * W, d.block_rows = br, d.total_rows = total;
            if (int rc = vmx_linear_launch(d, st)) return rc;
            const float *shared = nullptr;
            if (lc.shared_ff > 0) {
                VmxLinear su;
                su.A = m->h.p, su.a_f32 = f32, su.lda = W;
                su.W = L.sup.as<uint16_t>(), su.w_sn = W, su.w_sk = 1;
                su.C = m->sact.p, su.c_f32 = f32, su.ldc = lc.shared_ff;
                su.M = T, su.N = lc.shared_ff, su.K = W, su.exact = f32, su.epilogue = VMX_EP_RELU2;
                if (int rc = vmx_linear_launch(su, st)) return rc;
                VmxLinear sd;
                sd.A = m->sact.p, sd.a_f32 = f32, sd.lda = lc.shared_ff;
                sd.W = L.sdown.as<uint16_t>(), sd.w_sn = lc.shared_ff, sd.w_sk = 1;
                sd.C = m->sout.p, sd.c_f32 = 1, sd.ldc = W;
                sd.M = T, sd.N = W, sd.K = lc.shared_ff, sd.exact = f32;
                if (int rc = vmx_linear_launch(sd, st)) return rc;
                shared = m->sout.as<float>();
            }
            if (int rc = vmx_moe_combine_f32(x, m->ydown.as<float>(), inv, m->topw.as<float>(), k, shared, nullptr, 0, T, W, st)) return rc;
        }
        if (layer_trace)
            VMX_CHECK_HIP(hipMemcpyAsync(layer_trace + (size_t)li * T * W, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    }
    if (num_logit_rows > 0) {
        if (int rc = vmx_rms_norm_f32in(m->hsel.p, f32, x, logit_rows, m->final_norm.as<uint16_t>(), 0, W, c.norm_eps, num_logit_rows, st)) return rc;
        float *lg = logits ? logits : m->fused.as<float>();   // greedy ids only: the logits live in a workspace
        VMX_REQUIRE(logits || (size_t)num_logit_rows * c.vocab * 4 <= m->fused.bytes, "gesutar_forward: pass a logits buffer for %d rows",
                    num_logit_rows);
        VmxLinear hd;
        hd.A = m->hsel.p, hd.a_f32 = f32, hd.lda = W;
        hd.W = m->head.as<uint16_t>(), hd.w_sn = W, hd.w_sk = 1;
        hd.C = lg, hd.c_f32 = 1, hd.ldc = c.vocab;
        hd.M = num_logit_rows, hd.N = c.vocab, hd.K = W, hd.exact = f32;
        if (int rc = vmx_linear_launch(hd, st)) return rc;
        if (greedy_ids) {
            if (int rc = vmx_argmax_f32_rows(greedy_ids, m->argmax_keys.as<unsigned long long>(), lg, num_logit_rows, c.vocab, st)) return rc;
        }
    }
    return VMX_OK;
}
