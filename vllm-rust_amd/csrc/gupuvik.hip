// Whole-step executor of the Gupuvik decoder family: a stack of PARALLEL layers listed in the model's configuration,
//   h = x / sqrt(mean(x^2) + eps) * g                                   (one learned gain for the whole row)
//   x += sigmoid(R1 h + r1) * mixer(h) + sigmoid(R2 h + r2) * ff(h)     (element-wise gates; ff may be absent)
//   logits = head . norm(x)
// Mixer "attention" (window_attn.hip): grouped-query attention with biased projections, no rotation, a per-head temperature,
// tanh soft-capping, a sliding window that also keeps the sequence's first tokens, and a per-head sigmoid output gate; a layer may
// read the key/value cache of an earlier layer instead of projecting its own.  Mixer "channel_delta" (delta_rule.hip): short
// causal convolutions + SiLU on q, k, v, unit-vector q and k, a gated delta rule with one decay per key channel from a low-rank
// projection, per-head RMS norm and a low-rank sigmoid gate on the read-out.  Feed-forward: dense (tanh-GELU) or a mixture of
// SiLU-gated experts whose weights are the softmax over the chosen router logits.
//
// Every product that reads h (q, k, v, the head gates, the low-rank inner projections, both residual gates) is ONE linear whose
// f32 output row the other kernels address by column offset.  Tokens are packed as in the other packed executor; besides the paged
// key/value caches a sequence owns a STATE SLOT (convolution inputs and delta-rule memories of every recurrent layer), handed out
// by the caller.  The residual stream, norms, router, scores, softmax, decays, gates and the recurrence are f32 in both modes;
// VMX_BF16 rounds the operands of the linears and the cache rows to bf16, VMX_F32 multiplies in true f32 everywhere.
// The forward call allocates nothing, reads nothing back and is graph-capturable.
#include "vmx_kernels.h"
#include <math.h>
#include <algorithm>
#include <string>
#include <vector>

namespace {

using Buf = VmxBuf;

int pad8(int n) { return (n + 7) & ~7; }

struct Seg {       // where a checkpoint tensor lands: rows of the fused projection, or a buffer of its own
    Buf *buf = nullptr;
    size_t offset = 0, bytes = 0;
};

struct Layer {
    vmx_gupuvik_layer_config c;
    Buf norm1, wfused, bias, wo, temp, kcache, vcache;                       // both mixers / attention
    Buf conv_taps, a_log, dt_bias, onorm, wa2, wg2, conv_state, s_state;     // channel delta
    Buf wup, wdown, router, egu, edown;                                      // feed-forward
    int nf = 0, q_off = 0, k_off = 0, v_off = 0, g_off = 0, b_off = 0, a1_off = 0, g1_off = 0, rg1_off = 0, rg2_off = 0;
    std::vector<std::pair<std::string, Seg>> tensors;   // checkpoint name (without the layer prefix) -> destination
    std::vector<std::string> missing;
    void want(const std::string &name, Buf *b, size_t off, size_t bytes) {
        tensors.push_back({name, Seg{b, off, bytes}});
        missing.push_back(name);
    }
};

}  // namespace

struct vmx_gupuvik {
    vmx_gupuvik_config cfg;
    std::vector<Layer> layers;
    Buf embed, final_norm, head;
    std::vector<std::string> missing;
    Buf x, h, hsel, fused, attn, attn_ws, conv, dec, gate2, dro, argmax_keys, few_pairs, rlogits, topw, topi, sorted, blk_expert, total, inv, gu, act, ydown;
    bool f32() const { return cfg.dtype == VMX_F32; }
    size_t esz() const { return f32() ? 4 : 2; }
};

namespace {

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

int alloc_zero(Buf &b, size_t n) {
    if (int rc = b.alloc(n)) return rc;
    VMX_CHECK_HIP(hipMemset(b.p, 0, n ? n : 16));
    return VMX_OK;
}

}  // namespace

extern "C" int vmx_gupuvik_create(const vmx_gupuvik_config *cfg, const vmx_gupuvik_layer_config *layer_cfgs, vmx_gupuvik **out) {
    VMX_REQUIRE(cfg && layer_cfgs && out, "gupuvik_create: null pointer");
    const vmx_gupuvik_config &c = *cfg;
    VMX_REQUIRE(c.vocab >= 1 && c.width >= 1 && c.num_layers >= 1, "gupuvik_create: bad sizes (vocab %d, width %d, layers %d)", c.vocab, c.width,
                c.num_layers);
    VMX_REQUIRE(c.dtype == VMX_F32 || c.dtype == VMX_BF16, "gupuvik_create: dtype must be VMX_F32 or VMX_BF16");
    VMX_REQUIRE(c.block_size >= 1 && c.num_blocks >= 1 && c.max_tokens >= 1 && c.max_seqs >= 1 && c.state_slots >= 1,
                "gupuvik_create: bad cache / batch geometry");
    vmx_gupuvik *m = new vmx_gupuvik();
    m->cfg = c;
    m->layers.resize(c.num_layers);
    const size_t T = c.max_tokens, W = c.width, rows = (size_t)c.num_blocks * c.block_size;
    size_t attn_ws = 16, nf = 8, hv = 1, convc = 1, hd = 1, ne = 1, pairs = 0, cap = (size_t)VMX_MOE_FEW_PAIRS * 16, eff = 1, actn = 1;
    int rc = VMX_OK;
#define GA(buf, n)                        \
    do {                                  \
        if (!rc) rc = alloc_zero(buf, n); \
    } while (0)
#define BAD(...)                    \
    {                               \
        vmx_set_error(__VA_ARGS__); \
        rc = VMX_EINVAL;            \
        break;                      \
    }
    for (int li = 0; li < c.num_layers && !rc; li++) {
        Layer &L = m->layers[li];
        L.c = layer_cfgs[li];
        const vmx_gupuvik_layer_config &lc = L.c;
        if (lc.heads < 1 || lc.kv_heads < 1 || lc.heads % lc.kv_heads || lc.dim < 1 || lc.dim > 256 || lc.vdim < 1 || lc.vdim > 256)
            BAD("gupuvik_create: layer %d: bad head counts or sizes (heads %d, kv_heads %d, dim %d, vdim %d; sizes up to 256)", li, lc.heads,
                lc.kv_heads, lc.dim, lc.vdim);
        const bool ff = lc.mlp != VMX_MLP_NONE;
        const size_t H = lc.heads, G = lc.kv_heads, D = lc.dim, V = lc.vdim;
        int at = 0;
        auto seg = [&](int n) {
            const int o = at;
            at = pad8(at + n);
            return o;
        };
        L.want("norm1", &L.norm1, 0, 2);
        GA(L.norm1, 2);
        if (lc.mixer == VMX_MIXER_WINDOW_ATTENTION) {
            if (lc.window < 0 || lc.keep_first < 0 || lc.softcap < 0.f) BAD("gupuvik_create: layer %d: bad attention mask or soft cap", li);
            const bool own = lc.kv_from < 0;
            if (!own) {
                if (lc.kv_from >= li) BAD("gupuvik_create: layer %d reads the keys of layer %d, which does not run before it", li, lc.kv_from);
                const vmx_gupuvik_layer_config &sc = m->layers[lc.kv_from].c;
                if (sc.mixer != VMX_MIXER_WINDOW_ATTENTION || sc.kv_from >= 0 || sc.kv_heads != lc.kv_heads || sc.dim != lc.dim || sc.vdim != lc.vdim)
                    BAD("gupuvik_create: layer %d: layer %d holds no key/value cache of the same shape", li, lc.kv_from);
            }
            L.q_off = seg(H * D);
            if (own) L.k_off = seg(G * D), L.v_off = seg(G * V);
            L.g_off = seg(H);
            L.rg1_off = seg(W);
            if (ff) L.rg2_off = seg(W);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.bias, (size_t)L.nf * 2);
            GA(L.temp, H * 2);
            GA(L.wo, W * H * V * 2);
            L.want("mix.q", &L.wfused, (size_t)L.q_off * W * 2, H * D * W * 2);
            L.want("mix.q.b", &L.bias, (size_t)L.q_off * 2, H * D * 2);
            if (own) {
                GA(L.kcache, rows * G * D * m->esz());
                GA(L.vcache, rows * G * V * m->esz());
                L.want("mix.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
                L.want("mix.k.b", &L.bias, (size_t)L.k_off * 2, G * D * 2);
                L.want("mix.v", &L.wfused, (size_t)L.v_off * W * 2, G * V * W * 2);
                L.want("mix.v.b", &L.bias, (size_t)L.v_off * 2, G * V * 2);
            }
            attn_ws = std::max(attn_ws, vmx_window_attention_workspace_bytes((int)T, lc.heads, lc.vdim));
            L.want("mix.temp", &L.temp, 0, H * 2);
            L.want("mix.g", &L.wfused, (size_t)L.g_off * W * 2, H * W * 2);
            L.want("mix.o", &L.wo, 0, W * H * V * 2);
        } else if (lc.mixer == VMX_MIXER_CHANNEL_DELTA) {
            if (lc.conv_taps < 1 || lc.conv_taps > 64 || lc.decay_rank < 1 || lc.gate_rank < 1)
                BAD("gupuvik_create: layer %d: bad convolution length or projection ranks", li);
            const size_t C = 2 * G * D + H * V, n = lc.conv_taps;
            L.q_off = seg(2 * G * D + H * V);   // q | k | v stay adjacent: the convolution sees one run of channels
            L.k_off = L.q_off + G * D;
            L.v_off = L.k_off + G * D;
            L.b_off = seg(H);
            L.a1_off = seg(lc.decay_rank);
            L.g1_off = seg(lc.gate_rank);
            L.rg1_off = seg(W);
            if (ff) L.rg2_off = seg(W);
            L.nf = at;
            GA(L.wfused, (size_t)L.nf * W * 2);
            GA(L.bias, (size_t)L.nf * 2);
            GA(L.conv_taps, C * n * 2);
            GA(L.a_log, H * 2);
            GA(L.dt_bias, H * D * 2);
            GA(L.onorm, V * 2);
            GA(L.wa2, H * D * lc.decay_rank * 2);
            GA(L.wg2, H * V * lc.gate_rank * 2);
            GA(L.wo, W * H * V * 2);
            GA(L.conv_state, vmx_short_conv_state_bytes(c.state_slots, (int)C, lc.conv_taps));
            GA(L.s_state, vmx_gated_delta_rule_state_bytes(c.state_slots, lc.heads, lc.dim, lc.vdim));
            L.want("mix.q", &L.wfused, (size_t)L.q_off * W * 2, G * D * W * 2);
            L.want("mix.k", &L.wfused, (size_t)L.k_off * W * 2, G * D * W * 2);
            L.want("mix.v", &L.wfused, (size_t)L.v_off * W * 2, H * V * W * 2);
            L.want("mix.q.conv", &L.conv_taps, 0, G * D * n * 2);
            L.want("mix.k.conv", &L.conv_taps, G * D * n * 2, G * D * n * 2);
            L.want("mix.v.conv", &L.conv_taps, 2 * G * D * n * 2, H * V * n * 2);
            L.want("mix.b", &L.wfused, (size_t)L.b_off * W * 2, H * W * 2);
            L.want("mix.A_log", &L.a_log, 0, H * 2);
            L.want("mix.norm", &L.onorm, 0, V * 2);
            L.want("mix.a1", &L.wfused, (size_t)L.a1_off * W * 2, (size_t)lc.decay_rank * W * 2);
            L.want("mix.a2", &L.wa2, 0, H * D * lc.decay_rank * 2);
            L.want("mix.dt_bias", &L.dt_bias, 0, H * D * 2);
            L.want("mix.g1", &L.wfused, (size_t)L.g1_off * W * 2, (size_t)lc.gate_rank * W * 2);
            L.want("mix.g2", &L.wg2, 0, H * V * lc.gate_rank * 2);
            L.want("mix.o", &L.wo, 0, W * H * V * 2);
            convc = std::max(convc, C);
            hd = std::max(hd, H * D);
        } else {
            vmx_set_error("gupuvik_create: layer %d: unknown mixer kind %d", li, lc.mixer);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        L.want("rg1", &L.wfused, (size_t)L.rg1_off * W * 2, W * W * 2);
        L.want("rg1.b", &L.bias, (size_t)L.rg1_off * 2, W * 2);
        if (ff) {
            L.want("rg2", &L.wfused, (size_t)L.rg2_off * W * 2, W * W * 2);
            L.want("rg2.b", &L.bias, (size_t)L.rg2_off * 2, W * 2);
        }
        if (lc.mlp == VMX_MLP_DENSE_GELU) {
            if (lc.ff < 1) BAD("gupuvik_create: layer %d: bad feed-forward width", li);
            GA(L.wup, (size_t)lc.ff * W * 2);
            GA(L.wdown, (size_t)lc.ff * W * 2);
            L.want("mlp.up", &L.wup, 0, (size_t)lc.ff * W * 2);
            L.want("mlp.down", &L.wdown, 0, (size_t)lc.ff * W * 2);
            actn = std::max(actn, T * lc.ff);
        } else if (lc.mlp == VMX_MLP_GLU_MOE) {
            if (lc.experts < 1 || lc.experts > 256 || lc.top < 1 || lc.top > lc.experts || lc.expert_ff < 1)
                BAD("gupuvik_create: layer %d: bad mixture-of-experts sizes (1 .. 256 experts, top <= experts)", li);
            const size_t one = (size_t)lc.expert_ff * W * 2;
            GA(L.router, (size_t)lc.experts * W * 2);
            GA(L.egu, (size_t)lc.experts * 2 * one);
            GA(L.edown, (size_t)lc.experts * one);
            L.want("mlp.router", &L.router, 0, (size_t)lc.experts * W * 2);
            for (int e = 0; e < lc.experts; e++) {
                const std::string p = "mlp.e" + std::to_string(e) + ".";
                L.want(p + "gate", &L.egu, (size_t)e * 2 * one, one);   // per expert: gate rows, then up rows
                L.want(p + "up", &L.egu, (size_t)e * 2 * one + one, one);
                L.want(p + "down", &L.edown, (size_t)e * one, one);
            }
            ne = std::max(ne, (size_t)lc.experts);
            pairs = std::max(pairs, T * lc.top);
            cap = std::max(cap, T * lc.top + (size_t)lc.experts * 63);
            eff = std::max(eff, (size_t)lc.expert_ff);
        } else if (lc.mlp != VMX_MLP_NONE) {
            vmx_set_error("gupuvik_create: layer %d: unknown feed-forward kind %d", li, lc.mlp);
            rc = VMX_EUNSUPPORTED;
            break;
        }
        nf = std::max(nf, (size_t)L.nf);
        hv = std::max(hv, H * V);
    }
#undef BAD
    GA(m->embed, (size_t)c.vocab * W * 2);
    GA(m->final_norm, 2);
    GA(m->head, (size_t)c.vocab * W * 2);
    m->missing = {"embed", "final.norm", "head"};
    GA(m->x, T * W * 4);
    GA(m->h, T * W * m->esz());
    GA(m->hsel, T * W * m->esz());
    GA(m->fused, T * std::max(nf, (size_t)c.vocab) * 4);   // also the logits of a greedy-only step
    GA(m->attn, T * hv * m->esz());
    GA(m->attn_ws, attn_ws);   // key shares of attention launches with few rows
    GA(m->conv, T * convc * 4);
    GA(m->dec, T * hd * 4);
    GA(m->gate2, T * hv * 4);
    GA(m->dro, T * hv * 4);
    GA(m->argmax_keys, T * ((size_t)c.vocab / VMX_ARGMAX_CHUNK + 1) * 8);
    GA(m->few_pairs, (size_t)(2 * VMX_MOE_FEW_PAIRS * 16 + VMX_MOE_FEW_PAIRS + 1) * 4);
    GA(m->rlogits, T * ne * 4);
    GA(m->topw, (pairs + 1) * 4);
    GA(m->topi, (pairs + 1) * 4);
    GA(m->sorted, (cap + 1) * 4);
    GA(m->blk_expert, (cap / 16 + 2) * 4);
    GA(m->total, 16);
    GA(m->inv, (pairs + 1) * 4);
    GA(m->gu, (cap + 1) * 2 * eff * 4);
    GA(m->act, std::max((cap + 1) * eff, actn) * m->esz());
    GA(m->ydown, (cap + 1) * W * 4);
#undef GA
    if (!rc) {
        // decode steps with a handful of (token, slot) pairs skip the sort: pair p is its own 16-row block (row 16 p)
        const int FP = VMX_MOE_FEW_PAIRS;
        std::vector<int32_t> fp(2 * FP * 16 + FP + 1);
        for (int i = 0; i < FP * 16; i++) {
            fp[i] = i % 16 == 0 ? i / 16 : 0x7fffffff;              // gathered rows of the first product: pair index or padding
            fp[FP * 16 + i] = i % 16 == 0 ? i : 0x7fffffff;          // rows of the second product: themselves or padding
        }
        for (int p = 0; p < FP; p++) fp[2 * FP * 16 + p] = 16 * p;   // where pair p's result lies
        fp[2 * FP * 16 + FP] = 0x7fffffff;                           // "total rows": never cuts
        if (hipMemcpy(m->few_pairs.p, fp.data(), fp.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
            vmx_set_error("gupuvik_create: upload failed");
            rc = VMX_ELAUNCH;
        }
    }
    if (rc) {
        vmx_gupuvik_destroy(m);
        return rc;
    }
    *out = m;
    return VMX_OK;
}

extern "C" void vmx_gupuvik_destroy(vmx_gupuvik *m) {
    if (!m) return;
    for (Layer &L : m->layers)
        for (Buf *b : {&L.norm1, &L.wfused, &L.bias, &L.wo, &L.temp, &L.kcache, &L.vcache, &L.conv_taps, &L.a_log, &L.dt_bias, &L.onorm, &L.wa2, &L.wg2,
                       &L.conv_state, &L.s_state, &L.wup, &L.wdown, &L.router, &L.egu, &L.edown})
            b->release();
    for (Buf *b : {&m->embed, &m->final_norm, &m->head, &m->x, &m->h, &m->hsel, &m->fused, &m->attn, &m->attn_ws, &m->conv, &m->dec, &m->gate2, &m->dro,
                   &m->argmax_keys, &m->few_pairs, &m->rlogits, &m->topw, &m->topi, &m->sorted, &m->blk_expert, &m->total, &m->inv, &m->gu, &m->act,
                   &m->ydown})
        b->release();
    delete m;
}

extern "C" int vmx_gupuvik_load_tensor(vmx_gupuvik *m, const char *name, const void *data, size_t bytes, void *stream) {
    VMX_REQUIRE(m && name && (data || bytes == 0), "gupuvik_load_tensor: null pointer");
    hipStream_t st = vmx_stream(stream);
    const vmx_gupuvik_config &c = m->cfg;
    const size_t W = c.width;
    const std::string n(name);
    Seg dst;
    std::vector<std::string> *missing = &m->missing;
    std::string key = n;
    if (n == "embed") dst = Seg{&m->embed, 0, (size_t)c.vocab * W * 2};
    else if (n == "final.norm") dst = Seg{&m->final_norm, 0, 2};
    else if (n == "head") dst = Seg{&m->head, 0, (size_t)c.vocab * W * 2};
    else if (n.size() > 1 && n[0] == 'l' && isdigit((unsigned char)n[1])) {
        const size_t dot = n.find('.');
        VMX_REQUIRE(dot != std::string::npos, "gupuvik_load_tensor: unknown tensor `%s`", name);
        const int li = atoi(n.substr(1, dot - 1).c_str());
        VMX_REQUIRE(li >= 0 && li < c.num_layers, "gupuvik_load_tensor: `%s`: the model has %d layers", name, c.num_layers);
        Layer &L = m->layers[li];
        missing = &L.missing;
        key = n.substr(dot + 1);
        for (const auto &t : L.tensors)
            if (t.first == key) dst = t.second;
    }
    VMX_REQUIRE(dst.buf, "gupuvik_load_tensor: unknown tensor `%s`", name);
    VMX_REQUIRE(bytes == dst.bytes, "gupuvik_load_tensor: `%s`: expected %zu bytes of bf16, got %zu", name, dst.bytes, bytes);
    if (bytes > 0)
        if (int rc = upload(*dst.buf, dst.offset, data, bytes, st)) return rc;
    erase_name(*missing, key);
    return VMX_OK;
}

extern "C" int vmx_gupuvik_missing_tensors(const vmx_gupuvik *m) {
    if (!m) return -1;
    size_t n = m->missing.size();
    std::string first = m->missing.empty() ? "" : m->missing[0];
    for (size_t li = 0; li < m->layers.size(); li++) {
        const Layer &L = m->layers[li];
        if (first.empty() && !L.missing.empty()) first = "l" + std::to_string(li) + "." + L.missing[0];
        n += L.missing.size();
    }
    if (n) vmx_set_error("gupuvik: %zu tensors not loaded, first `%s`", n, first.c_str());
    return (int)n;
}

extern "C" int vmx_gupuvik_forward(vmx_gupuvik *m, const int32_t *tokens, const int32_t *positions, const int32_t *slots, const int32_t *seq_ids,
                                   int num_tokens, const int32_t *block_tables, int num_seqs, int max_blocks_per_seq, const int32_t *seq_starts,
                                   const int32_t *state_slots, const int32_t *logit_rows, int num_logit_rows, float *logits, int32_t *greedy_ids,
                                   float *layer_trace, void *stream) {
    VMX_REQUIRE(m && tokens && positions && slots && seq_ids && block_tables && seq_starts && state_slots, "gupuvik_forward: null pointer");
    const vmx_gupuvik_config &c = m->cfg;
    VMX_REQUIRE(num_tokens >= 1 && num_tokens <= c.max_tokens, "gupuvik_forward: %d tokens, the model was created for at most %d", num_tokens,
                c.max_tokens);
    VMX_REQUIRE(num_seqs >= 1 && num_seqs <= c.max_seqs && max_blocks_per_seq >= 1, "gupuvik_forward: bad sequence count or block-table shape");
    VMX_REQUIRE(num_logit_rows >= 0 && num_logit_rows <= num_tokens && (num_logit_rows == 0 || (logit_rows && (logits || greedy_ids))),
                "gupuvik_forward: bad logit rows");
    if (vmx_gupuvik_missing_tensors(m) != 0) return VMX_EINVAL;
    hipStream_t st = vmx_stream(stream);
    const int T = num_tokens, W = c.width, f32 = m->f32() ? 1 : 0;
    const int cdt = f32 ? VMX_F32 : VMX_BF16;
    float *x = m->x.as<float>(), *fused = m->fused.as<float>();
    if (int rc = vmx_embed_scaled_f32(x, m->embed.as<uint16_t>(), tokens, T, W, c.vocab, (float)c.embed_scale, st)) return rc;
    for (int li = 0; li < c.num_layers; li++) {
        Layer &L = m->layers[li];
        const vmx_gupuvik_layer_config &lc = L.c;
        const int H = lc.heads, G = lc.kv_heads, D = lc.dim, V = lc.vdim, nf = L.nf;
        if (int rc = vmx_rms_norm_f32in(m->h.p, f32, x, nullptr, L.norm1.as<uint16_t>(), 1, W, c.norm_eps, T, st)) return rc;
        {   // everything that reads h: projections, head gates, low-rank inner projections, both residual gates
            VmxLinear p;
            p.A = m->h.p, p.a_f32 = f32, p.lda = W;
            p.W = L.wfused.as<uint16_t>(), p.w_sn = W, p.w_sk = 1, p.bias = L.bias.as<uint16_t>();
            p.C = fused, p.c_f32 = 1, p.ldc = nf;
            p.M = T, p.N = nf, p.K = W, p.exact = f32;
            if (int rc = vmx_linear_launch(p, st)) return rc;
        }
        if (lc.mixer == VMX_MIXER_WINDOW_ATTENTION) {
            if (lc.kv_from < 0)
                if (int rc = vmx_kv_cache_write_f32(fused + L.k_off, nf, fused + L.v_off, nf, slots, L.kcache.p, L.vcache.p, cdt, T, G * D, G * V, st))
                    return rc;
            Layer &S = lc.kv_from < 0 ? L : m->layers[lc.kv_from];
            if (int rc = vmx_window_attention(m->attn.p, cdt, fused + L.q_off, nf, S.kcache.p, S.vcache.p, cdt, block_tables, max_blocks_per_seq,
                                              seq_ids, positions, L.temp.as<uint16_t>(), fused + L.g_off, nf, lc.scale, lc.softcap, lc.window,
                                              lc.keep_first, T, H, G, D, V, c.block_size, seq_starts, num_seqs, m->attn_ws.p, m->attn_ws.bytes, st))
                return rc;
        } else {
            const int C = 2 * G * D + H * V;
            {   // decay logits: second half of the low-rank projection
                VmxLinear a;
                a.A = fused + L.a1_off, a.a_f32 = 1, a.lda = nf;
                a.W = L.wa2.as<uint16_t>(), a.w_sn = lc.decay_rank, a.w_sk = 1;
                a.C = m->dec.p, a.c_f32 = 1, a.ldc = (int64_t)H * D;
                a.M = T, a.N = H * D, a.K = lc.decay_rank, a.exact = f32;
                if (int rc = vmx_linear_launch(a, st)) return rc;
            }
            {   // output gate logits
                VmxLinear g;
                g.A = fused + L.g1_off, g.a_f32 = 1, g.lda = nf;
                g.W = L.wg2.as<uint16_t>(), g.w_sn = lc.gate_rank, g.w_sk = 1;
                g.C = m->gate2.p, g.c_f32 = 1, g.ldc = (int64_t)H * V;
                g.M = T, g.N = H * V, g.K = lc.gate_rank, g.exact = f32;
                if (int rc = vmx_linear_launch(g, st)) return rc;
            }
            float *cv = m->conv.as<float>();
            if (int rc = vmx_short_conv_silu(fused + L.q_off, nf, L.conv_taps.as<uint16_t>(), L.conv_state.as<float>(), cv, C, positions, seq_ids,
                                             seq_starts, state_slots, T, C, lc.conv_taps, D, 2 * G, G, 1e-6f, 1.0f / sqrtf((float)D), st))
                return rc;
            if (int rc = vmx_short_conv_state_update(fused + L.q_off, nf, L.conv_state.as<float>(), positions, seq_starts, state_slots, num_seqs, C,
                                                     lc.conv_taps, st))
                return rc;
            if (int rc = vmx_delta_rule_gates(m->dec.as<float>(), (int64_t)H * D, L.a_log.as<uint16_t>(), L.dt_bias.as<uint16_t>(), fused + L.b_off,
                                              nf, T, H, D, st))
                return rc;
            if (int rc = vmx_gated_delta_rule(m->dro.as<float>(), (int64_t)H * V, cv, C, cv + G * D, C, cv + 2 * G * D, C, m->dec.as<float>(),
                                              (int64_t)H * D, fused + L.b_off, nf, L.s_state.as<float>(), positions, seq_starts, state_slots,
                                              num_seqs, H, G, D, V, st))
                return rc;
            if (int rc = vmx_head_rms_gate(m->attn.p, cdt, m->dro.as<float>(), (int64_t)H * V, L.onorm.as<uint16_t>(), m->gate2.as<float>(),
                                           (int64_t)H * V, c.norm_eps, T, H, V, st))
                return rc;
        }
        {   // x += sigmoid(gate 1) * W_o mixer
            VmxLinear o;
            o.A = m->attn.p, o.a_f32 = f32, o.lda = (int64_t)H * V;
            o.W = L.wo.as<uint16_t>(), o.w_sn = (int64_t)H * V, o.w_sk = 1;
            o.C = x, o.c_f32 = 1, o.ldc = W;
            o.M = T, o.N = W, o.K = H * V, o.exact = f32;
            o.epilogue = VMX_EP_ADD_MUL_SIGMOID, o.aux = fused + L.rg1_off, o.ldaux = nf;
            if (int rc = vmx_linear_launch(o, st)) return rc;
        }
        if (lc.mlp == VMX_MLP_DENSE_GELU) {
            VmxLinear u;
            u.A = m->h.p, u.a_f32 = f32, u.lda = W;
            u.W = L.wup.as<uint16_t>(), u.w_sn = W, u.w_sk = 1;
            u.C = m->act.p, u.c_f32 = f32, u.ldc = lc.ff;
            u.M = T, u.N = lc.ff, u.K = W, u.exact = f32, u.epilogue = VMX_EP_GELU_TANH;
            if (int rc = vmx_linear_launch(u, st)) return rc;
            VmxLinear d;
            d.A = m->act.p, d.a_f32 = f32, d.lda = lc.ff;
            d.W = L.wdown.as<uint16_t>(), d.w_sn = lc.ff, d.w_sk = 1;
            d.C = x, d.c_f32 = 1, d.ldc = W;
            d.M = T, d.N = W, d.K = lc.ff, d.exact = f32;
            d.epilogue = VMX_EP_ADD_MUL_SIGMOID, d.aux = fused + L.rg2_off, d.ldaux = nf;
            if (int rc = vmx_linear_launch(d, st)) return rc;
        } else if (lc.mlp == VMX_MLP_GLU_MOE) {
            const int E = lc.experts, k = lc.top, ff = lc.expert_ff, pairs = T * k, FP = VMX_MOE_FEW_PAIRS;
            VmxLinear r;   // router logits: always a true f32 product
            r.A = m->h.p, r.a_f32 = f32, r.lda = W;
            r.W = L.router.as<uint16_t>(), r.w_sn = W, r.w_sk = 1;
            r.C = m->rlogits.p, r.c_f32 = 1, r.ldc = E;
            r.M = T, r.N = E, r.K = W, r.exact = 1;
            if (int rc = vmx_linear_launch(r, st)) return rc;
            // the largest `top` logits; softmax over all experts renormalised over the chosen = softmax over the chosen logits
            if (int rc = vmx_topk_softmax(m->rlogits.p, VMX_F32, m->topw.as<float>(), m->topi.as<int32_t>(), T, E, k, 1, 0, stream)) return rc;
            const bool few = pairs <= FP;   // every pair its own block: no sort
            const int br = few ? 16 : (pairs >= 32 * E ? 64 : 16);
            const int cap = few ? pairs * 16 : pairs + E * (br - 1);
            const int32_t *fp = m->few_pairs.as<int32_t>();
            const int32_t *up_rows = few ? fp : m->sorted.as<int32_t>(), *down_rows = few ? fp + FP * 16 : nullptr;
            const int32_t *blk = few ? m->topi.as<int32_t>() : m->blk_expert.as<int32_t>();
            const int32_t *total = few ? fp + 2 * FP * 16 + FP : m->total.as<int32_t>();
            const int32_t *inv = few ? fp + 2 * FP * 16 : m->inv.as<int32_t>();
            if (!few) {
                if (int rc = vmx_moe_align_block_size(m->topi.as<int32_t>(), m->sorted.as<int32_t>(), m->blk_expert.as<int32_t>(),
                                                      m->total.as<int32_t>(), pairs, E, br, cap, stream))
                    return rc;
                if (int rc = vmx_moe_inverse(m->inv.as<int32_t>(), m->sorted.as<int32_t>(), m->total.as<int32_t>(), pairs, cap, st)) return rc;
            }
            VmxLinear u;   // gate | up of the pairs' rows in one product
            u.A = m->h.p, u.a_f32 = f32, u.lda = W;
            u.W = L.egu.as<uint16_t>(), u.w_sn = W, u.w_sk = 1;
            u.C = m->gu.p, u.c_f32 = 1, u.ldc = 2 * ff;
            u.M = cap, u.N = 2 * ff, u.K = W, u.exact = f32;
            u.row_ids = up_rows, u.row_div = k, u.row_limit = pairs;
            u.block_expert = blk, u.expert_stride = (int64_t)2 * ff * W, u.block_rows = br, u.total_rows = total;
            if (int rc = vmx_linear_launch(u, st)) return rc;
            if (int rc = vmx_glu_silu_rows(m->act.p, f32, m->gu.as<float>(), cap, ff, st)) return rc;
            VmxLinear d;
            d.A = m->act.p, d.a_f32 = f32, d.lda = ff;
            d.W = L.edown.as<uint16_t>(), d.w_sn = ff, d.w_sk = 1;
            d.C = m->ydown.p, d.c_f32 = 1, d.ldc = W;
            d.M = cap, d.N = W, d.K = ff, d.exact = f32;
            d.row_ids = down_rows, d.row_div = 1, d.row_limit = cap;
            d.block_expert = blk, d.expert_stride = (int64_t)ff * W, d.block_rows = br, d.total_rows = total;
            if (int rc = vmx_linear_launch(d, st)) return rc;
            if (int rc = vmx_moe_combine_f32(x, m->ydown.as<float>(), inv, m->topw.as<float>(), k, nullptr, fused + L.rg2_off, nf, T, W, st)) return rc;
        }
        if (layer_trace)
            VMX_CHECK_HIP(hipMemcpyAsync(layer_trace + (size_t)li * T * W, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    }
    if (num_logit_rows > 0) {
        if (int rc = vmx_rms_norm_f32in(m->hsel.p, f32, x, logit_rows, m->final_norm.as<uint16_t>(), 1, W, c.norm_eps, num_logit_rows, st)) return rc;
        float *lg = logits ? logits : fused;   // greedy ids only: the logits live in a workspace
        VmxLinear hd;
        hd.A = m->hsel.p, hd.a_f32 = f32, hd.lda = W;
        hd.W = m->head.as<uint16_t>(), hd.w_sn = W, hd.w_sk = 1;
        hd.C = lg, hd.c_f32 = 1, hd.ldc = c.vocab;
        hd.M = num_logit_rows, hd.N = c.vocab, hd.K = W, hd.exact = f32;
        if (int rc = vmx_linear_launch(hd, st)) return rc;
        if (greedy_ids)
            if (int rc = vmx_argmax_f32_rows(greedy_ids, m->argmax_keys.as<unsigned long long>(), lg, num_logit_rows, c.vocab, st)) return rc;
    }
    return VMX_OK;
}
