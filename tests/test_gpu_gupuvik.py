"""Gupuvik on the GPU against the float64 oracle (tests/gupuvik_oracle.py): every mechanism alone (window attention with the
kept first tokens, short convolution and gated delta rule with carried state, the read-out norm, the router), then the executor
through the engine's step function under different cuttings of the same tokens (whole prompts, token-by-token decoding, portions
down to two tokens, unequal batches, recycled cache blocks and state slots), window / page / first-token edges with inputs that
make a single key stand out, other sizes, and greedy generation through the scheduler.  Small random models built here; float32
mode is held to 2e-4 of the logits' spread, bfloat16 mode to 4e-2."""
import json
import math
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def gpu():
    import torch
    import vllm_rust_amd as vmx
    assert torch.cuda.is_available()
    vmx.init(0)
    return vmx, torch


def attn_layer(**kw):
    from vllm_rust_amd.gupuvik import GupuvikLayerSpec
    d = dict(mixer="attention", heads=4, kv_heads=2, dim=12, vdim=20, window=6, keep_first=2, scale=0.3, softcap=8.0, mlp="moe", experts=6,
             top=2, expert_ff=24)
    d.update(kw)
    return GupuvikLayerSpec(**d)


def delta_layer(**kw):
    from vllm_rust_amd.gupuvik import GupuvikLayerSpec
    d = dict(mixer="channel_delta", heads=4, kv_heads=2, dim=10, vdim=36, conv=3, decay_rank=5, gate_rank=6, mlp="dense", ff=56)
    d.update(kw)
    return GupuvikLayerSpec(**d)


def small_spec(layers=None, **kw):
    from vllm_rust_amd.gupuvik import GupuvikSpec
    layers = layers or [delta_layer(), attn_layer(), delta_layer(mlp="moe", experts=5, top=3, expert_ff=16), attn_layer(kv_from=1, window=9, keep_first=0),
                        attn_layer(mlp=None, window=0, softcap=0.0, heads=2, kv_heads=2)]
    d = dict(vocab=61, width=40, layers=layers, norm_eps=1e-5, embed_scale=2.5)
    d.update(kw)
    return GupuvikSpec(**d)


def sure_routing(spec):
    """The same model with every expert chosen (top = experts): long bfloat16 runs, where some router decision among hundreds is
    always a close call, then test everything but the choice."""
    import dataclasses
    return dataclasses.replace(spec, layers=[dataclasses.replace(l, top=l.experts) if l.mlp == "moe" else l for l in spec.layers])


def build(spec, dtype="float32", seed=0, tweak=None, block_size=4, num_blocks=96, max_tokens=320, max_seqs=6):
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.gupuvik import GupuvikForCausalLM, synthetic_weights
    ck = synthetic_weights(spec, seed)
    if tweak:
        tweak(ck)
    model = GupuvikForCausalLM(spec, dtype=dtype, block_size=block_size, num_blocks=num_blocks, max_tokens=max_tokens, max_seqs=max_seqs)
    model.load_state(ck)
    return model, Engine(model), {k: v.double() for k, v in ck.items()}


def rel_err(got, want):
    """Difference of two logits arrays, row means removed, relative to the spread of the expected rows (worst row)."""
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = g - w
    d = d - d.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (w.std(-1) + 1e-12)).max())


TOL = {"float32": 2e-4, "bfloat16": 4e-2}


def tokens_for(spec, n, seed, weights=None):
    """n random token ids.  With the model's weights: the first draw on which no router decision of the oracle is a close call
    (relative gap above 1 %), since a decision that bf16 rounding can flip says nothing about the kernels."""
    from tests import gupuvik_oracle as orc
    for attempt in range(200):
        toks = np.random.default_rng(seed + 1000 * attempt).integers(0, spec.vocab, n).tolist()
        if weights is None or orc.min_router_margin(toks, weights, spec.to_config()) > 0.01:
            return toks
    raise AssertionError("no token draw with safe router margins")


def oracle_logits(spec, weights, toks):
    from tests import gupuvik_oracle as orc
    return orc.forward(toks, weights, spec.to_config()).numpy()


def feed(engine, seq_id, toks, cuts, finish=True):
    """Feed toks to one sequence in pieces of the given sizes (the last size repeats); logits of every position."""
    out, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        lg, _, _ = engine.step([(seq_id, toks[at:at + n], list(range(n)))])
        out.append(lg.cpu().numpy())
        at += n
        i += 1
    if finish:
        engine.finish(seq_id)
    return np.concatenate(out)


# ----------------------------------------------------------------------------- mechanisms alone

def _window_attention_op(torch, q, k, v, temp, gate, scale, cap, window, keep, block_size, dtype, seed=1, runs=False):
    """vmx_window_attention for ONE sequence whose blocks are scattered over a larger cache; every position is a query.
    runs: tell the operator which rows form a sequence (it then takes its matrix-core form where the sizes and the cache allow);
    runs == "split": also hand it a workspace, so that it deals the keys of a run to several workgroups and merges."""
    from vllm_rust_amd._lib import check, lib
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    nb = (T + block_size - 1) // block_size
    perm = np.random.default_rng(seed).permutation(nb + 7)[:nb].astype(np.int32)
    cdt = torch.float32 if dtype == 0 else torch.bfloat16
    kc = torch.full(((nb + 7) * block_size, G * D), float("nan"), dtype=torch.float32)
    vc = torch.full(((nb + 7) * block_size, G * V), float("nan"), dtype=torch.float32)
    pos = np.arange(T)
    rows = perm[pos // block_size] * block_size + pos % block_size
    kc[rows], vc[rows] = k.reshape(T, G * D).float(), v.reshape(T, G * V).float()
    kc, vc = kc.to(cdt).cuda(), vc.to(cdt).cuda()
    out = torch.empty((T, H * V), dtype=torch.float32, device="cuda")
    qd = q.reshape(T, H * D).float().cuda()
    bt, sid, pid = torch.from_numpy(perm[None]).cuda(), torch.zeros(T, dtype=torch.int32, device="cuda"), torch.arange(T, dtype=torch.int32, device="cuda")
    td = None if temp is None else temp.to(torch.bfloat16).cuda()
    gd = None if gate is None else gate.float().cuda()
    st = torch.tensor([0, T], dtype=torch.int32, device="cuda")
    ws = torch.empty(lib.vmx_window_attention_workspace_bytes(T, H, V) // 4, dtype=torch.float32, device="cuda")
    check(lib.vmx_window_attention(out.data_ptr(), 0, qd.data_ptr(), H * D, kc.data_ptr(), vc.data_ptr(), dtype, bt.data_ptr(), nb, sid.data_ptr(),
                                   pid.data_ptr(), None if td is None else td.data_ptr(), None if gd is None else gd.data_ptr(), H, scale, cap, window,
                                   keep, T, H, G, D, V, block_size, st.data_ptr() if runs else None, 1 if runs else 0,
                                   ws.data_ptr() if runs == "split" else None, ws.numel() * 4, None))
    torch.cuda.synchronize()
    return out.cpu().double().view(T, H, V)


def _attention_want(torch, q, k, v, temp, gate, scale, cap, window, keep):
    from tests import gupuvik_oracle as orc
    T, H, D = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=torch.float64)
    for h in range(H):
        for i in range(T):
            js = [j for j in range(T) if orc.visible(i, j, window if window else T + 1, keep)]
            s = torch.stack([q[i, h] @ k[j, h // (H // G)] for j in js]) * scale * (1.0 if temp is None else temp[h])
            if cap:
                s = cap * torch.tanh(s / cap)
            p = torch.softmax(s, 0)
            out[i, h] = (p[:, None] * torch.stack([v[j, h // (H // G)] for j in js])).sum(0) * (1.0 if gate is None else torch.sigmoid(gate[i, h]))
    return out


@pytest.mark.parametrize("H,G,D,V,window,keep,cap,bs", [(4, 2, 12, 20, 6, 2, 8.0, 4), (3, 1, 7, 70, 0, 0, 0.0, 3), (2, 2, 16, 16, 70, 5, 30.0, 16),
                                                       (6, 3, 33, 130, 5, 9, 2.0, 1), (1, 1, 64, 64, 1, 0, 0.0, 8), (2, 1, 8, 8, 3, 40, 5.0, 4),
                                                       (8, 2, 40, 24, 40, 7, 15.0, 16), (16, 2, 128, 128, 100, 0, 0.0, 16), (3, 3, 72, 24, 0, 0, 9.0, 2),
                                                       (6, 2, 136, 40, 20, 30, 0.0, 4)])
@pytest.mark.parametrize("dtype,runs", [(0, False), (1, False), (1, True), (1, "split")])
def test_window_attention_operator(gpu, H, G, D, V, window, keep, cap, bs, dtype, runs):
    vmx, torch = gpu
    g = torch.Generator().manual_seed(H * 100 + D)
    T = 150
    rnd = lambda *s: torch.randn(s, generator=g).to(torch.bfloat16).double()   # noqa: E731  (values both cache types hold exactly)
    q, k, v = rnd(T, H, D), rnd(T, G, D), rnd(T, G, V)
    temp, gate = (1.0 + 0.3 * torch.randn(H, generator=g)).to(torch.bfloat16).double(), torch.randn((T, H), generator=g).double()
    got = _window_attention_op(torch, q, k, v, temp, gate, 0.4, cap, window, keep, bs, dtype, runs=runs)
    want = _attention_want(torch, q, k, v, temp, gate, 0.4, cap, window, keep)
    assert float((got - want).abs().max()) <= 2e-5 * max(1.0, float(want.abs().max()))   # q holds bf16 values: both forms are exact in the operands


@pytest.mark.parametrize("dtype,runs", [(0, False), (1, False), (1, True), (1, "split")])
@pytest.mark.parametrize("bs", [4, 16])
def test_window_attention_needle_at_every_edge(gpu, dtype, runs, bs):
    """One key carries a score far above all others and a value nobody else has.  A query sees it exactly while it is inside the
    window or among the kept first tokens; the query positions sit on both sides of each edge and the needle on block borders."""
    vmx, torch = gpu
    T, D, V, window, keep = 700, 16, 8, 64, 3
    for needle in (0, 2, 3, 4, 15, 16, 17, 63, 64, 300):
        g = torch.Generator().manual_seed(needle)
        q = 0.05 * torch.randn((T, 1, D), generator=g).double()
        k = 0.05 * torch.randn((T, 1, D), generator=g).double()
        v = torch.zeros((T, 1, V), dtype=torch.float64)
        v[:, 0, 0] = 1.0
        q[:, 0, 0], k[needle, 0, 0], v[needle, 0, :] = 4.0, 4.0, torch.tensor([0.0, 9.0] + [0.0] * (V - 2))
        q, k = q.to(torch.bfloat16).double(), k.to(torch.bfloat16).double()
        got = _window_attention_op(torch, q, k, v, None, None, 1.0, 0.0, window, keep, bs, dtype, seed=needle, runs=runs)
        for i in (needle, needle + 1, needle + window - 2, needle + window - 1, needle + window, needle + window + 1, T - 1):
            if needle <= i < T:
                seen = needle < keep or i - needle < window
                assert (float(got[i, 0, 1]) > 8.0) == seen, (needle, i, float(got[i, 0, 1]))
                assert abs(float(got[i, 0, 0])) < 0.1 if seen else abs(float(got[i, 0, 0]) - 1.0) < 1e-5


def _packed(torch, lens, starts_pos):
    pos = np.concatenate([np.arange(p, p + n) for n, p in zip(lens, starts_pos)]).astype(np.int32)
    sid = np.concatenate([np.full(n, i) for i, n in enumerate(lens)]).astype(np.int32)
    st = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()   # noqa: E731
    return dev(pos), dev(sid), dev(st)


@pytest.mark.parametrize("taps,C,group,ug,sg", [(4, 50, 10, 3, 2), (2, 130, 1, 0, 0), (1, 24, 8, 3, 0), (7, 96, 70, 1, 1)])
def test_short_convolution_carries_its_state(gpu, taps, C, group, ug, sg):
    """Two sequences fed in unequal portions (down to one token, shorter than the filter) against the whole-sequence convolution."""
    from tests import gupuvik_oracle as orc
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(taps * 10 + C)
    lens = [23, 9]
    xs = [torch.randn((n, C), generator=g).double() for n in lens]
    w = torch.randn((C, taps), generator=g).to(torch.bfloat16)
    want = []
    for x in xs:
        y = orc.causal_conv_silu(x, w.double())
        for u in range(ug):
            y[:, u * group:(u + 1) * group] = orc.unit(y[:, u * group:(u + 1) * group]) * (0.5 if u < sg else 1.0)
        want.append(y)
    state = torch.full((5, max(taps - 1, 1), C), float("nan"), dtype=torch.float32, device="cuda")   # slots hold garbage at first
    slots = torch.tensor([3, 1], dtype=torch.int32, device="cuda")
    got = [[], []]
    at = [0, 0]
    wd = w.cuda()
    for cut in ([1, 2], [2, 1], [1, 1], [5, 3], [3, 2], [11, 0]):
        idx = [i for i in (0, 1) if cut[i] > 0]
        ls = [cut[i] for i in idx]
        pos, sid, st = _packed(torch, ls, [at[i] for i in idx])
        x = torch.cat([xs[i][at[i]:at[i] + cut[i]] for i in idx]).float().cuda()
        y = torch.empty_like(x)
        sl = slots[idx].contiguous()
        check(lib.vmx_short_conv_silu(x.data_ptr(), C, wd.data_ptr(), state.data_ptr(), y.data_ptr(), C, pos.data_ptr(), sid.data_ptr(),
                                      st.data_ptr(), sl.data_ptr(), x.shape[0], C, taps, group, ug, sg, 1e-6, 0.5, None))
        check(lib.vmx_short_conv_state_update(x.data_ptr(), C, state.data_ptr(), pos.data_ptr(), st.data_ptr(), sl.data_ptr(), len(idx), C, taps, None))
        torch.cuda.synchronize()
        o = 0
        for i in idx:
            got[i].append(y[o:o + cut[i]].cpu().double())
            o += cut[i]
            at[i] += cut[i]
    for i in (0, 1):
        assert float((torch.cat(got[i]) - want[i]).abs().max()) <= 1e-5


@pytest.mark.parametrize("H,Hk,D,V", [(4, 2, 10, 36), (2, 2, 64, 32), (3, 1, 100, 7), (1, 1, 200, 65), (6, 6, 8, 128)])
def test_gated_delta_rule_operator(gpu, H, Hk, D, V):
    """Portions of two sequences through recycled state slots against the plain scan over whole sequences."""
    from tests import gupuvik_oracle as orc
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(H + D + V)
    lens = [37, 12]
    seqs = []
    for n in lens:
        q = orc.unit(torch.randn((n, Hk, D), generator=g).double()) * D ** -0.5
        k = orc.unit(torch.randn((n, Hk, D), generator=g).double())
        v = torch.randn((n, H, V), generator=g).double()
        beta = torch.rand((n, H), generator=g).double()
        decay = torch.exp(-0.3 * torch.rand((n, H, D), generator=g).double())
        seqs.append((q, k, v, beta, decay))
    want = [orc.delta_rule_scan(*s) for s in seqs]
    nbytes = lib.vmx_gated_delta_rule_state_bytes(4, H, D, V)
    state = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    slots = torch.tensor([2, 0], dtype=torch.int32, device="cuda")
    got, at = [[], []], [0, 0]
    for cut in ([1, 12], [1, 0], [2, 0], [9, 0], [24, 0]):
        idx = [i for i in (0, 1) if cut[i] > 0]
        ls = [cut[i] for i in idx]
        pos, _, st = _packed(torch, ls, [at[i] for i in idx])
        part = [torch.cat([seqs[i][j][at[i]:at[i] + cut[i]] for i in idx]).float().cuda().flatten(1).contiguous() for j in range(5)]
        o = torch.empty((sum(ls), H * V), dtype=torch.float32, device="cuda")
        sl = slots[idx].contiguous()
        check(lib.vmx_gated_delta_rule(o.data_ptr(), H * V, part[0].data_ptr(), Hk * D, part[1].data_ptr(), Hk * D, part[2].data_ptr(), H * V,
                                       part[4].data_ptr(), H * D, part[3].data_ptr(), H, state.data_ptr(), pos.data_ptr(), st.data_ptr(), sl.data_ptr(),
                                       len(idx), H, Hk, D, V, None))
        torch.cuda.synchronize()
        a = 0
        for i in idx:
            got[i].append(o[a:a + cut[i]].cpu().double().view(cut[i], H, V))
            a += cut[i]
            at[i] += cut[i]
    for i in (0, 1):
        assert float((torch.cat(got[i]) - want[i]).abs().max()) <= 2e-5 * max(1.0, float(want[i].abs().max()))


def test_delta_gates_and_read_out_norm(gpu):
    from tests import gupuvik_oracle as orc
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(3)
    T, H, D, V = 9, 3, 10, 36
    z = (3 * torch.randn((T, H * D), generator=g)).float()
    b = torch.randn((T, H), generator=g).float()
    a_log, dt_bias = torch.randn(H, generator=g).to(torch.bfloat16), torch.randn(H * D, generator=g).to(torch.bfloat16)
    want = torch.exp(-torch.exp(a_log.double())[None, :, None] * orc.softplus(z.double() + dt_bias.double()).view(T, H, D))
    zc, bc, ad, dd = z.cuda(), b.cuda(), a_log.cuda(), dt_bias.cuda()
    check(lib.vmx_delta_rule_gates(zc.data_ptr(), H * D, ad.data_ptr(), dd.data_ptr(), bc.data_ptr(), H, T, H, D, None))
    torch.cuda.synchronize()
    assert float((zc.cpu().double().view(T, H, D) - want).abs().max()) <= 1e-6
    assert float((bc.cpu().double() - torch.sigmoid(b.double())).abs().max()) <= 1e-6
    o, gate, w = torch.randn((T, H, V), generator=g).float(), torch.randn((T, H, V), generator=g).float(), torch.randn(V, generator=g).to(torch.bfloat16)
    y = torch.empty((T, H * V), dtype=torch.float32, device="cuda")
    oc, wc, gc = o.cuda(), w.cuda(), gate.cuda()
    check(lib.vmx_head_rms_gate(y.data_ptr(), 0, oc.data_ptr(), H * V, wc.data_ptr(), gc.data_ptr(), H * V, 1e-5, T, H, V, None))
    torch.cuda.synchronize()
    od = o.double()
    want = od / torch.sqrt((od * od).mean(-1, keepdim=True) + 1e-5) * w.double() * torch.sigmoid(gate.double())
    assert float((y.cpu().double().view(T, H, V) - want).abs().max()) <= 1e-5


@pytest.mark.parametrize("E,top", [(6, 2), (8, 8), (5, 1), (200, 7)])
def test_router_is_a_softmax_over_the_chosen_logits(gpu, E, top):
    from tests import gupuvik_oracle as orc
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(E)
    h, w = torch.randn((19, 16), generator=g).double(), {"router": (3 * torch.randn((E, 16), generator=g)).double()}
    idx, wt, z = orc.route(h, w, "", top)
    zc = z.float().cuda()
    wo, io = torch.empty((19, top), dtype=torch.float32, device="cuda"), torch.empty((19, top), dtype=torch.int32, device="cuda")
    check(lib.vmx_topk_softmax(zc.data_ptr(), 0, wo.data_ptr(), io.data_ptr(), 19, E, top, 1, 0, None))
    torch.cuda.synchronize()
    assert io.cpu().tolist() == idx.tolist()
    assert np.allclose(wo.cpu().numpy(), wt.numpy(), rtol=1e-5, atol=1e-7)


# ----------------------------------------------------------------------------- the executor through the engine

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_against_the_oracle(gpu, dtype):
    from tests import gupuvik_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 40, 1, w if dtype == "bfloat16" else None)
    lg, _, trace = eng.step([("a", toks, list(range(len(toks))))], layer_trace=True)
    want, layers = orc.forward(toks, w, spec.to_config(), return_layers=True)
    for i in range(len(spec.layers)):
        scale = float(layers[i].abs().max())
        assert float((trace[i].cpu().double() - layers[i]).abs().max()) <= (5e-5 if dtype == "float32" else 4e-2) * scale, f"layer {i}"
    assert rel_err(lg.cpu().numpy(), want.numpy()) <= TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompt_equals_decoding_equals_portions(gpu, dtype):
    """The same tokens as one prompt, token by token, and in portions of 2 / 3 / 7 / 16 (then single tokens): every cutting
    against the oracle, and in float32 against each other to rounding."""
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 61, 2, w if dtype == "bfloat16" else None)
    want = oracle_logits(spec, w, toks)
    runs = {cut: feed(eng, f"s{cut}", toks, cut) for cut in ((61,), (1,), (2,), (3,), (7,), (16, 1), (30, 2, 1))}
    for cut, got in runs.items():
        assert rel_err(got, want) <= TOL[dtype], cut
    if dtype == "float32":
        for cut, got in runs.items():
            assert rel_err(got, runs[(61,)]) <= 2e-5, cut


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batches_against_each_request_alone(gpu, dtype):
    """Prompts of 1, 5, 19 and 42 tokens start together, then decode together; the shorter requests end earlier, and a new
    request takes over a finished one's blocks and state slot while the others go on."""
    vmx, torch = gpu
    spec = small_spec() if dtype == "float32" else sure_routing(small_spec())
    model, eng, w = build(spec, dtype)
    lens, total = [1, 5, 19, 42], [6, 13, 40, 60]
    toks = [tokens_for(spec, n, 10 + i, w if dtype == "bfloat16" else None) for i, n in enumerate(total)]
    want = [oracle_logits(spec, w, t) for t in toks]
    got = [[] for _ in toks]
    lg, _, _ = eng.step([(i, toks[i][:lens[i]], list(range(lens[i]))) for i in range(4)])
    at, o = list(lens), 0
    for i in range(4):
        got[i].append(lg[o:o + lens[i]].cpu().numpy())
        o += lens[i]
    late = tokens_for(spec, 25, 77, w if dtype == "bfloat16" else None)
    late_got, late_at = [], 0
    while any(at[i] < total[i] for i in range(4)) or late_at < len(late):
        live = [i for i in range(4) if at[i] < total[i]]
        entries = [(i, [toks[i][at[i]]], [0]) for i in live]
        if len(live) < 4 and late_at < len(late):
            n = 3 if late_at == 0 else 1     # joins as a short prompt, then decodes with the rest
            entries.append(("late", late[late_at:late_at + n], list(range(n))))
        lg, _, _ = eng.step(entries)
        lg = lg.cpu().numpy()
        for j, i in enumerate(live):
            got[i].append(lg[j:j + 1])
            at[i] += 1
            if at[i] == total[i]:
                eng.finish(i)
        if len(entries) > len(live):
            late_got.append(lg[len(live):])
            late_at += len(entries[-1][1])
    for i in range(4):
        assert rel_err(np.concatenate(got[i]), want[i]) <= TOL[dtype], i
    assert rel_err(np.concatenate(late_got), oracle_logits(spec, w, late)) <= TOL[dtype]


def test_blocks_and_state_slots_are_reused(gpu):
    """More requests than state slots or blocks for all of them at once, one after another and interleaved: what a finished
    request leaves in its blocks and its slot must not reach the next owner."""
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, "float32", num_blocks=24, max_seqs=2)
    for r in range(5):
        a, b = tokens_for(spec, 30 + r, 20 + r), tokens_for(spec, 9 + 2 * r, 40 + r)
        ga, gb = [], []
        for lo in range(0, 40, 5):
            entries = [(n, t[lo:lo + 5], list(range(len(t[lo:lo + 5])))) for n, t in (("a", a), ("b", b)) if t[lo:lo + 5]]
            if not entries:
                break
            lg, _, _ = eng.step(entries)
            lg = lg.cpu().numpy()
            na = len(a[lo:lo + 5])
            ga.append(lg[:na])
            gb.append(lg[na:])
        eng.finish("b")
        eng.finish("a")
        assert rel_err(np.concatenate(ga), oracle_logits(spec, w, a)) <= TOL["float32"], r
        assert rel_err(np.concatenate(gb), oracle_logits(spec, w, b)) <= TOL["float32"], r
    assert len(eng.blocks.free) == 24 and sorted(eng.states.free) == [0, 1]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_window_and_first_token_edges_in_prompts_and_decoding(gpu, dtype):
    """Windows of 1 .. 17 keys with 0 .. 5 kept first tokens and page sizes that put the edges on and off page borders; with so few
    visible keys every one of them carries weight, so a window that is one key off shows at once.  130 tokens as a prompt + decoding."""
    vmx, torch = gpu
    for window, keep, bs in ((1, 0, 4), (4, 4, 4), (5, 1, 3), (8, 5, 8), (17, 2, 16), (3, 0, 1)):
        spec = small_spec(layers=[attn_layer(window=window, keep_first=keep, mlp=None), delta_layer(mlp=None),
                                  attn_layer(window=window + 1, keep_first=max(keep - 1, 0), mlp="dense", ff=24), attn_layer(kv_from=0, window=2 * window, keep_first=keep + 1, mlp=None)])
        model, eng, w = build(spec, dtype, seed=window, block_size=bs, num_blocks=200 if bs == 1 else 64)
        toks = tokens_for(spec, 130, window)
        want = oracle_logits(spec, w, toks)
        assert rel_err(feed(eng, "p", toks, (90, 1)), want) <= TOL[dtype], (window, keep, bs)
        assert rel_err(feed(eng, "q", toks, (2, 1)), want) <= TOL[dtype], (window, keep, bs)
        model.close()


def test_attention_reaches_far_keys_and_the_first_tokens(gpu):
    """Near-one-hot attention at model level: the key projection is made to answer the query projection for ONE early token, so
    that the logits late in a long sequence depend on whether that token is still visible (kept first tokens: yes; outside the
    window and not kept: no).  The oracle sees the same weights."""
    vmx, torch = gpu
    spec = small_spec(layers=[attn_layer(window=50, keep_first=3, softcap=30.0, scale=1.0, mlp=None, heads=2, kv_heads=1, dim=16, vdim=16)])

    def tweak(ck):
        ck["l0.mix.q"] *= 4.0
        ck["l0.mix.k"] *= 4.0
    model, eng, w = build(spec, "float32", tweak=tweak, block_size=16, num_blocks=40, max_tokens=400)
    toks = tokens_for(spec, 300, 5)
    want = oracle_logits(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, (300,)), want) <= TOL["float32"]
    assert rel_err(feed(eng, "b", toks, (260, 1)), want) <= TOL["float32"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(gpu, dtype):
    vmx, torch = gpu
    spec = small_spec() if dtype == "float32" else sure_routing(small_spec())
    model, eng, w = build(spec, dtype, max_tokens=64)
    toks = tokens_for(spec, 200, 9, w if dtype == "bfloat16" else None)
    got = feed(eng, "a", toks, (3, 1))
    assert rel_err(got, oracle_logits(spec, w, toks)) <= TOL[dtype]


SIZES = [
    dict(width=44, layers=[delta_layer(heads=1, kv_heads=1, dim=7, vdim=5, conv=1, decay_rank=1, gate_rank=3, mlp=None),
                           attn_layer(heads=1, kv_heads=1, dim=5, vdim=3, window=0, keep_first=0, softcap=0.0, experts=4, top=4, expert_ff=9)]),
    dict(width=24, vocab=17, layers=[attn_layer(heads=6, kv_heads=6, dim=8, vdim=8, window=7, keep_first=9, mlp="dense", ff=8),
                                     attn_layer(heads=6, kv_heads=6, dim=8, vdim=8, kv_from=0, window=1, keep_first=0, mlp=None),
                                     attn_layer(heads=6, kv_heads=6, dim=8, vdim=8, kv_from=0, window=0, keep_first=0, experts=1, top=1, expert_ff=40)]),
    dict(width=64, layers=[delta_layer(heads=2, kv_heads=1, dim=72, vdim=70, conv=6, decay_rank=16, gate_rank=8, mlp="moe", experts=9, top=2, expert_ff=8),
                           delta_layer(heads=8, kv_heads=8, dim=4, vdim=4, conv=2, decay_rank=3, gate_rank=1)]),
    dict(width=32, embed_scale=1.0, norm_eps=1e-3, layers=[attn_layer(heads=8, kv_heads=2, dim=20, vdim=72, window=1000, keep_first=1000, mlp="dense", ff=100),
                                                           delta_layer(heads=3, kv_heads=3, dim=130, vdim=12, conv=4, decay_rank=7, gate_rank=7, mlp=None)]),
]


@pytest.mark.parametrize("case", range(len(SIZES)))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_other_sizes(gpu, case, dtype):
    """One head, equal head counts, sizes that are not multiples of 8, a filter of one tap, rank 1, top = experts, one expert,
    layers without feed-forward, several layers on one cache, no window, no soft cap, windows larger than the sequence."""
    vmx, torch = gpu
    spec = small_spec(**SIZES[case])
    model, eng, w = build(spec, dtype, seed=case, block_size=[1, 2, 8, 5][case], num_blocks=160)
    toks = tokens_for(spec, 45, case, w if dtype == "bfloat16" else None)
    want = oracle_logits(spec, w, toks)
    assert rel_err(feed(eng, "a", toks, (45,)), want) <= TOL[dtype]
    assert rel_err(feed(eng, "b", toks, (20, 2, 1)), want) <= TOL[dtype]


def random_spec(seed):
    """A model drawn at random: layer order, head counts, sizes (half of them multiples of 8, which the matrix-core attention
    takes), windows, kept tokens, caps, shared caches, filter lengths, ranks, feed-forward kinds."""
    rng = np.random.default_rng(seed)
    pick = lambda *a: a[int(rng.integers(len(a)))]   # noqa: E731
    size = lambda lo, hi: 8 * int(rng.integers(1, hi // 8 + 1)) if rng.random() < 0.5 else int(rng.integers(lo, hi + 1))   # noqa: E731

    def ff():
        kind = pick(None, "dense", "moe", "moe")
        if kind == "dense":
            return dict(mlp="dense", ff=int(rng.integers(4, 70)))
        if kind == "moe":
            e = int(rng.integers(1, 10))
            return dict(mlp="moe", experts=e, top=int(rng.integers(1, e + 1)), expert_ff=int(rng.integers(4, 40)))
        return dict(mlp=None)
    layers, own = [], []
    for i in range(int(rng.integers(2, 6))):
        kv = pick(1, 2, 3)
        heads = kv * pick(1, 2, 3, 4, 8)
        if rng.random() < 0.5:
            layers.append(delta_layer(heads=heads, kv_heads=kv, dim=size(3, 80), vdim=size(3, 72), conv=int(rng.integers(1, 6)),
                                      decay_rank=int(rng.integers(1, 13)), gate_rank=int(rng.integers(1, 13)), **ff()))
            continue
        mask = dict(window=pick(0, int(rng.integers(1, 40))), keep_first=int(rng.integers(0, 7)), softcap=pick(0.0, 5.0, 20.0), scale=pick(0.1, 0.3, 1.0))
        if own and rng.random() < 0.4:
            src = own[int(rng.integers(len(own)))]
            l = layers[src]
            layers.append(attn_layer(heads=l.kv_heads * pick(1, 3, 4), kv_heads=l.kv_heads, dim=l.dim, vdim=l.vdim, kv_from=src, **mask, **ff()))
        else:
            layers.append(attn_layer(heads=heads, kv_heads=kv, dim=size(3, 72), vdim=size(3, 72), **mask, **ff()))
            own.append(i)
    return small_spec(layers=layers, width=pick(24, 40, 52, 64), vocab=int(rng.integers(20, 90)), embed_scale=pick(1.0, 2.0, 4.0), norm_eps=pick(1e-6, 1e-5))


@pytest.mark.parametrize("seed", range(24))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_configurations(gpu, seed, dtype):
    """Two requests of unequal length start together and decode together, a third is fed in portions: against the oracle."""
    vmx, torch = gpu
    spec = random_spec(seed)
    if dtype == "bfloat16":
        spec = sure_routing(spec)
    model, eng, w = build(spec, dtype, seed=seed, block_size=[1, 2, 4, 8, 16][seed % 5], num_blocks=400 if seed % 5 == 0 else 120)
    a, b, c = tokens_for(spec, 62, seed), tokens_for(spec, 33, seed + 50), tokens_for(spec, 41, seed + 90)
    wa, wb = oracle_logits(spec, w, a), oracle_logits(spec, w, b)
    lg, _, _ = eng.step([("a", a[:47], list(range(47))), ("b", b[:18], list(range(18)))])
    ga, gb = [lg[:47].cpu().numpy()], [lg[47:].cpu().numpy()]
    for p in range(15):
        lg, _, _ = eng.step([("b", [b[18 + p]], [0]), ("a", [a[47 + p]], [0])])
        gb.append(lg[:1].cpu().numpy())
        ga.append(lg[1:].cpu().numpy())
    assert rel_err(np.concatenate(ga), wa) <= TOL[dtype] and rel_err(np.concatenate(gb), wb) <= TOL[dtype]
    eng.finish("a")
    assert rel_err(feed(eng, "c", c, (17, 5, 2, 1)), oracle_logits(spec, w, c)) <= TOL[dtype]
    model.close()


@pytest.mark.parametrize("seed", [100, 101, 102, 103])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_configurations_on_long_sequences(gpu, seed, dtype):
    """The same kind of model with windows of up to 300 keys and 700 tokens: key tiles, key shares and staging rounds all
    wrap several times; 620 tokens as a prompt next to a short request, then 80 decoded."""
    import dataclasses
    vmx, torch = gpu
    spec = random_spec(seed)
    spec = dataclasses.replace(spec, layers=[dataclasses.replace(l, window=8 * l.window, keep_first=4 * l.keep_first) if l.mixer == "attention" else l
                                             for l in spec.layers])
    if dtype == "bfloat16":
        spec = sure_routing(spec)
    model, eng, w = build(spec, dtype, seed=seed, block_size=16, num_blocks=64, max_tokens=700)
    a, b = tokens_for(spec, 700, seed), tokens_for(spec, 30, seed + 1)
    want = oracle_logits(spec, w, a)
    lg, _, _ = eng.step([("b", b[:9], []), ("a", a[:620], list(range(620)))])
    got = [lg.cpu().numpy()]
    for p in range(80):
        entries = [("a", [a[620 + p]], [0])] + ([("b", [b[9 + p]], [])] if 9 + p < len(b) else [])
        got.append(eng.step(entries)[0].cpu().numpy())
    assert rel_err(np.concatenate(got), want) <= TOL[dtype]
    model.close()


def test_long_prompt_whole_and_in_portions(gpu):
    """16 500 tokens with four experts per token: more (token, expert) pairs than one launch axis of 65 535 takes.  The whole prompt
    in one step gives the same last rows as portions of 4 096 (the plain oracle is too slow for this length and checks the first
    300 tokens of the same model)."""
    vmx, torch = gpu
    spec = small_spec(width=32, layers=[delta_layer(heads=2, kv_heads=1, dim=8, vdim=8, mlp="moe", experts=4, top=4, expert_ff=8),
                                        attn_layer(heads=2, kv_heads=1, dim=8, vdim=8, window=32, keep_first=2, experts=4, top=4, expert_ff=8)])
    n = 16500
    model, eng, w = build(spec, "float32", block_size=16, num_blocks=2 * (n // 16 + 2), max_tokens=n, max_seqs=2)
    toks = np.random.default_rng(0).integers(0, spec.vocab, n).tolist()
    want_rows = [n - 3, n - 2, n - 1]
    whole, _, _ = eng.step([("a", toks, want_rows)])
    parts = None
    for lo in range(0, n, 4096):
        piece = toks[lo:lo + 4096]
        lg, _, _ = eng.step([("b", piece, [r - lo for r in want_rows if lo <= r < lo + len(piece)])])
        parts = lg if lg is not None else parts
    assert torch.isfinite(whole).all() and rel_err(parts.cpu().numpy(), whole.cpu().numpy()) <= 2e-5
    eng.finish("a")
    eng.finish("b")
    short = toks[:300]
    assert rel_err(feed(eng, "c", short, (300,))[-2:], oracle_logits(spec, w, short)[-2:]) <= TOL["float32"]


def test_mixture_steps_on_both_sides_of_the_sort_threshold(gpu):
    """Decode batches whose (token, expert) pairs stay below and go above the count from which they are sorted into expert blocks
    give the rows the same logits."""
    vmx, torch = gpu
    spec = small_spec(layers=[attn_layer(experts=6, top=3, expert_ff=16), delta_layer(mlp="moe", experts=6, top=3, expert_ff=16)])
    model, eng, w = build(spec, "float32", max_seqs=8, num_blocks=128)
    toks = [tokens_for(spec, 12, 50 + i) for i in range(8)]
    want = [oracle_logits(spec, w, t) for t in toks]
    for group in (range(0, 6), range(6, 8)):     # 18 pairs per decode step (sorted), then 6 (unsorted); prompts: more
        eng.step([(i, toks[i][:4], []) for i in group])
        for p in range(4, 12):
            lg, _, _ = eng.step([(i, [toks[i][p]], [0]) for i in group])
            for j, i in enumerate(group):
                assert rel_err(lg[j:j + 1].cpu().numpy(), want[i][p:p + 1]) <= TOL["float32"]
    for i in range(8):
        eng.finish(i)
    lg, _, _ = eng.step([(f"x{i}", toks[i], [11]) for i in range(8)][:6])
    for i in range(6):
        assert rel_err(lg[i:i + 1].cpu().numpy(), want[i][11:12]) <= TOL["float32"]


def test_greedy_generation_through_the_scheduler(gpu):
    """Engine.generate (scheduler, prompt portions, joint decoding, block pressure) against greedy decoding with the oracle."""
    from vllm_rust_amd.engine import SamplingParams
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, "float32", num_blocks=40, max_seqs=3, max_tokens=48)
    prompts = [tokens_for(spec, n, 60 + n) for n in (3, 17, 30, 8, 1)]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=6), prefill_chunk=7)
    for p, got in zip(prompts, outs):
        seq = list(p)
        for t in got:
            lg = oracle_logits(spec, w, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(np.argmax(lg)) == t or top2[1] - top2[0] < 1e-3 * (np.abs(lg).max() + 1e-9)
            seq.append(t)
    assert len(eng.blocks.free) == 40 and len(eng.states.free) == 3
    sampled = eng.generate(prompts[:2], SamplingParams(temperature=0.8, top_k=5, top_p=0.9, max_new_tokens=4, seed=1))
    assert all(len(o) == 4 and all(0 <= t < spec.vocab for t in o) for o in sampled)


def _write_checkpoint(tmp_path, spec, seed):
    from safetensors.torch import save_file
    from vllm_rust_amd.gupuvik import synthetic_weights
    ck = synthetic_weights(spec, seed)
    save_file({k: v.contiguous() for k, v in ck.items()}, str(tmp_path / "model.safetensors"))
    cfg = spec.to_config()
    for e in cfg["layers"]:                      # a checkpoint states no ranks: they are the shapes of its tensors
        e["mixer"].pop("decay_rank", None)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    return {k: v.double() for k, v in ck.items()}


def test_registry_loads_a_checkpoint_directory(gpu, tmp_path):
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.models import architecture_of, load_model
    vmx, torch = gpu
    spec = small_spec()
    w = _write_checkpoint(tmp_path, spec, 4)
    assert architecture_of(tmp_path) == "Gupuvik"
    for dtype in ("float32", "bfloat16"):
        model = load_model(tmp_path, dtype=dtype, max_tokens=64, max_seqs=4, block_size=8)
        assert [(l.decay_rank, l.gate_rank) for l in model.spec.layers if l.mixer == "channel_delta"] == [(5, 6), (5, 6)]
        toks = tokens_for(spec, 20, 3, w if dtype == "bfloat16" else None)
        assert rel_err(feed(Engine(model), "a", toks, (20,)), oracle_logits(spec, w, toks)) <= TOL[dtype]


def test_trace_replay_tool(gpu, tmp_path):
    """bin/trace_run as a subprocess: two requests start together, decode together, one ends early; rows against the oracle."""
    vmx, torch = gpu
    spec = small_spec()
    mdir, out = tmp_path / "m", tmp_path / "out"
    mdir.mkdir()
    w = _write_checkpoint(mdir, spec, 6)
    a, b = tokens_for(spec, 12, 1), tokens_for(spec, 7, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:9], "want": [0, 8]}, {"id": "b", "tokens": b[:6], "want": [5]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[9:10], "want": []}, {"id": "b", "tokens": b[6:7], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:11], "want": [0]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[11:12], "want": [0]}], "end": ["a"]}]
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(mdir), "--dtype", "float32", "--out", str(out), "--max-tokens", "64"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = oracle_logits(spec, w, a), oracle_logits(spec, w, b)
    rd = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, spec.vocab)   # noqa: E731
    assert rel_err(rd(0), np.stack([wa[0], wa[8], wb[5]])) <= TOL["float32"]
    assert rel_err(rd(1), wb[6:7]) <= TOL["float32"] and rel_err(rd(2), wa[10:11]) <= TOL["float32"] and rel_err(rd(3), wa[11:12]) <= TOL["float32"]


def test_generation_tool(gpu, tmp_path):
    """bin/generate as a subprocess (registry, scheduler, greedy ids from the executor) against greedy decoding with the oracle."""
    vmx, torch = gpu
    spec = small_spec()
    w = _write_checkpoint(tmp_path, spec, 8)
    prompts = [tokens_for(spec, 9, 3), tokens_for(spec, 2, 4)]
    p = subprocess.run([sys.executable, str(ROOT / "bin" / "generate"), "--model", str(tmp_path), "--dtype", "float32", "--max-new-tokens", "4",
                        "--max-tokens", "64", "--prefill-chunk", "4"] + [a for q in prompts for a in ("--prompt", ",".join(map(str, q)))],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    outs = [[int(t) for t in line.split(",")] for line in p.stdout.strip().splitlines()]
    assert len(outs) == 2
    for q, got in zip(prompts, outs):
        seq = list(q)
        for t in got:
            lg = oracle_logits(spec, w, seq)[-1]
            top2 = np.sort(lg)[-2:]
            assert int(np.argmax(lg)) == t or top2[1] - top2[0] < 1e-3 * (np.abs(lg).max() + 1e-9)
            seq.append(t)
