"""Gesutar on the GPU against the float64 oracle (tests/gesutar_oracle.py): every mechanism alone, then the executor through the
engine's step function under different cuttings of the same tokens (whole prompts, token-by-token decoding, portions, mixed
batches, recycled cache blocks), window and page edges with weights that make a single key stand out, odd sizes, and greedy
generation through the scheduler.  Small random models built here; float32 mode is held to 2e-4 of the logits' spread,
bfloat16 mode to 4e-2."""
import dataclasses
import math

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch
    import vllm_rust_amd as vmx
    assert torch.cuda.is_available()
    vmx.init(0)
    return vmx, torch


def small_spec(**kw):
    from vllm_rust_amd.gesutar import GesutarLayerSpec, GesutarSpec
    lk = dict(heads=3, dim=16, rot_dim=8, vdim=24, kv_rank=40, window=12, rot_dims=8, rot_base=5000.0, scale=0.2, mlp="moe", experts=6,
              top=2, groups=3, keep_groups=2, expert_ff=24, shared_ff=16, router_scale=1.5)
    lk.update(kw.pop("layer", {}))
    layers = kw.pop("layers", None) or [GesutarLayerSpec(**lk), GesutarLayerSpec(**lk)]
    d = dict(vocab=89, width=48, layers=layers, norm_eps=1e-5, embed_scale=3.0, bigram_buckets=53, bigram_mul_prev=13, bigram_mul_cur=5)
    d.update(kw)
    return GesutarSpec(**d)


def build(spec, dtype="float32", seed=0, tweak=None, block_size=4, num_blocks=64, max_tokens=256):
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.gesutar import GesutarForCausalLM, synthetic_weights
    ck = synthetic_weights(spec, seed)
    if tweak:
        tweak(ck)
    model = GesutarForCausalLM(spec, dtype=dtype, block_size=block_size, num_blocks=num_blocks, max_tokens=max_tokens, max_seqs=16)
    model.load_state(ck)
    return model, Engine(model), {k: v.double() for k, v in ck.items()}


def rel_err(got, want):
    """Difference of two logits arrays, row means removed, relative to the spread of the expected rows (worst row)."""
    g, w = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = g - w
    d = d - d.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (w.std(-1) + 1e-12)).max())


TOL = {"float32": 2e-4, "bfloat16": 4e-2}


def tokens_for(spec, n, seed, weights=None, extra=0):
    """n random token ids (+ `extra` more).  With the model's weights: the first draw on which no router decision of the oracle is
    a close call (relative gap above 1 %), since a decision that bf16 rounding can flip says nothing about the kernels."""
    from tests import gesutar_oracle as orc
    for attempt in range(300):
        toks = np.random.default_rng(seed + 1000 * attempt).integers(0, spec.vocab, n + extra).tolist()
        if weights is None:
            return toks
        margins = []
        orc.forward(spec, weights, toks, margins=margins)
        if not margins or min(margins) > 0.01:
            return toks
    raise AssertionError("no token draw with safe router margins")


# ----------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("E,G,keep,top", [(12, 3, 2, 4), (8, 1, 1, 2), (16, 4, 4, 3), (6, 6, 2, 1), (1, 1, 1, 1), (192, 8, 3, 6)])
def test_grouped_router(gpu, E, G, keep, top):
    from tests import gesutar_oracle as orc
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(E * 7 + G)
    z = (torch.randn((37, E), generator=g) * 2).float()
    ids, w = orc.grouped_router(z, E, G, keep, top, 2.5)
    zc = z.cuda()
    wo = torch.empty((37, top), dtype=torch.float32, device="cuda")
    io = torch.empty((37, top), dtype=torch.int32, device="cuda")
    check(lib.vmx_grouped_topk_router(zc.data_ptr(), wo.data_ptr(), io.data_ptr(), 37, E, top, G, keep, 2.5, None))
    torch.cuda.synchronize()
    assert io.cpu().tolist() == ids
    assert np.allclose(wo.cpu().numpy(), w.numpy(), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("M,N,K", [(1, 70, 40), (5, 64, 64), (17, 33, 100), (100, 130, 72), (64, 9, 7)])
@pytest.mark.parametrize("exact", [1, 0])
def test_linear_any_shape(gpu, M, N, K, exact):
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(M + N + K)
    x = torch.randn((M, K), generator=g)
    w = (torch.randn((N, K), generator=g) / math.sqrt(K)).to(torch.bfloat16)
    wc = w.cuda()
    for xdt in (torch.float32, torch.bfloat16):
        xc = x.to(xdt).cuda()
        y = torch.empty((M, N), dtype=torch.float32, device="cuda")
        check(lib.vmx_linear_bf16w(y.data_ptr(), 0, xc.data_ptr(), 0 if xdt == torch.float32 else 1, wc.data_ptr(), M, N, K, exact, None))
        torch.cuda.synchronize()
        xin = xc.cpu().double() if exact else xc.cpu().to(torch.bfloat16).double()
        want = xin @ w.double().T
        assert float((y.cpu().double() - want).abs().max()) <= 2e-5 * max(1.0, float(want.abs().max()))


def test_linear_rows_do_not_depend_on_the_batch(gpu):
    """A row multiplied alone has the same bits as the same row inside a larger call of the same family (up to 16 rows: the
    streaming kernel; more: the tiled kernels), and the two families agree to rounding."""
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(5)
    x = torch.randn((100, 96), generator=g).to(torch.bfloat16).cuda()
    w = (torch.randn((80, 96), generator=g) / 10).to(torch.bfloat16).cuda()

    def run(rows, exact):
        xin = x[rows].contiguous()
        y = torch.empty((xin.shape[0], 80), dtype=torch.float32, device="cuda")
        check(lib.vmx_linear_bf16w(y.data_ptr(), 0, xin.data_ptr(), 1, w.data_ptr(), xin.shape[0], 80, 96, exact, None))
        torch.cuda.synchronize()
        return y
    for exact in (0, 1):
        one, few = run(slice(77, 78), exact), run(slice(70, 86), exact)
        many, most = run(slice(40, 100), exact), run(slice(0, 100), exact)
        assert torch.equal(one[0], few[7]) and torch.equal(many[37], most[77])
        assert float((one[0] - most[77]).abs().max()) <= 1e-5


def _attention_op(torch, q_abs, q_rot, cache_rows, window, sink, scale, block_size, dtype, shuffle_seed=1, workspace=True):
    """Run vmx_latent_attention for ONE sequence whose key j has the cache row cache_rows[j]; every position is a query.
    The sequence's blocks are scattered over a larger cache."""
    from vllm_rust_amd._lib import check, lib
    T, H, R = q_abs.shape
    rd = q_rot.shape[2]
    nb = (T + block_size - 1) // block_size
    perm = np.random.default_rng(shuffle_seed).permutation(nb + 5)[:nb].astype(np.int32)
    cache = torch.full(((nb + 5) * block_size, R + rd), float("nan"), dtype=torch.float32)
    for j in range(T):
        cache[perm[j // block_size] * block_size + j % block_size] = cache_rows[j]
    cdt = 0 if dtype == "float32" else 1
    cache = cache.cuda() if cdt == 0 else cache.to(torch.bfloat16).cuda()
    out = torch.empty((T, H, R), dtype=torch.float32, device="cuda")
    bt = torch.from_numpy(perm[None, :]).cuda()
    sid = torch.zeros(T, dtype=torch.int32, device="cuda")
    pos = torch.arange(T, dtype=torch.int32, device="cuda")
    sk = None if sink is None else sink.to(torch.bfloat16).cuda()
    q_rot_dev = q_rot.float().cuda() if rd else torch.zeros(1, device="cuda")
    nbytes = lib.vmx_latent_attention_workspace_bytes(T, H, R, window, nb, block_size) if workspace else 0
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
    q_abs_dev = q_abs.float().cuda()                  # every device operand stays referenced until the kernel has run
    check(lib.vmx_latent_attention(out.data_ptr(), q_abs_dev.data_ptr(), q_rot_dev.data_ptr(), cache.data_ptr(), cdt,
                                   bt.data_ptr(), nb, sid.data_ptr(), pos.data_ptr(), None if sk is None else sk.data_ptr(), scale, window, T, H, R,
                                   rd, block_size, ws.data_ptr() if nbytes else None, nbytes, None))
    torch.cuda.synchronize()
    return out.cpu().double()


def _attention_ref(torch, q_abs, q_rot, rows, window, sink, scale):
    from tests import gesutar_oracle as orc
    T, H, R = q_abs.shape
    pos = torch.arange(T)
    gap = pos[:, None] - pos[None, :]
    allowed = (gap >= 0) & ((gap < window) if window > 0 else (gap >= 0))
    out = torch.zeros(T, H, R, dtype=torch.float64)
    for h in range(H):
        sc = (q_abs[:, h].double() @ rows[:, :R].double().T + q_rot[:, h].double() @ rows[:, R:].double().T) * scale
        out[:, h] = orc.softmax_with_sink(sc, allowed, None if sink is None else sink[h].double()) @ rows[:, :R].double()
    return out


@pytest.mark.parametrize("window,use_sink,R,rd,bs", [(9, True, 24, 6, 4), (0, False, 70, 0, 16), (300, True, 130, 16, 8), (1, True, 8, 2, 3),
                                                     (70, True, 88, 24, 16), (0, True, 40, 8, 4), (129, False, 512, 64, 16), (64, True, 136, 0, 8)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_latent_attention_op(gpu, window, use_sink, R, rd, bs, dtype):
    vmx, torch = gpu
    g = torch.Generator().manual_seed(R + window)
    T, H = 330, 2          # more keys than one 256-key pass of the kernel
    rows = torch.randn((T, R + rd), generator=g)
    if dtype == "bfloat16":
        rows = rows.to(torch.bfloat16).float()
    q_abs, q_rot = torch.randn((T, H, R), generator=g), torch.randn((T, H, rd), generator=g)
    sink = torch.randn(H, generator=g).to(torch.bfloat16).float() if use_sink else None
    # the matrix-core form (bf16 cache, sizes in multiples of 8) takes the queries as bf16
    mfma = dtype == "bfloat16" and R % 8 == 0 and rd % 8 == 0
    if mfma:
        q_abs, q_rot = q_abs.to(torch.bfloat16).float(), q_rot.to(torch.bfloat16).float()
    want = _attention_ref(torch, q_abs, q_rot, rows, window, sink, 0.3 / math.sqrt(R / 24))
    for ws in (True, False):                          # with key partitions, and as one walk over all keys
        got = _attention_op(torch, q_abs, q_rot, rows, window, sink, 0.3 / math.sqrt(R / 24), bs, dtype, workspace=ws)
        assert float((got - want).abs().max()) <= (1e-4 if mfma else 2e-5)


@pytest.mark.parametrize("H", [1, 3, 8, 16, 20])
def test_latent_attention_mixed_sequences_in_one_tile(gpu, H):
    """Packed decode tokens of several sequences with different lengths: with fewer than 16 heads one 16-row tile of the
    matrix-core form holds tokens of different sequences; with more than 16 a token spans two tiles."""
    from vllm_rust_amd._lib import check, lib
    vmx, torch = gpu
    g = torch.Generator().manual_seed(H)
    R, rd, bs, window = 32, 8, 4, 21
    lens = [5, 70, 1, 33, 22, 64, 65]
    S, maxb = len(lens), 20
    cache = torch.randn((S * maxb * bs, R + rd), generator=g).to(torch.bfloat16)
    bt = torch.randperm(S * maxb, generator=g).to(torch.int32).reshape(S, maxb)
    q_abs = torch.randn((S, H, R), generator=g).to(torch.bfloat16).float()
    q_rot = torch.randn((S, H, rd), generator=g).to(torch.bfloat16).float()
    sink = torch.randn(H, generator=g).to(torch.bfloat16)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    out = torch.empty((S, H, R), dtype=torch.float32, device="cuda")
    nbytes = lib.vmx_latent_attention_workspace_bytes(S, H, R, window, maxb, bs)
    ws = torch.empty(max(nbytes, 4), dtype=torch.uint8, device="cuda")
    dev = [t.cuda() for t in (q_abs, q_rot, cache, bt, torch.arange(S, dtype=torch.int32), pos, sink)]      # kept alive over the launch
    check(lib.vmx_latent_attention(out.data_ptr(), dev[0].data_ptr(), dev[1].data_ptr(), dev[2].data_ptr(), 1, dev[3].data_ptr(), maxb,
                                   dev[4].data_ptr(), dev[5].data_ptr(), dev[6].data_ptr(), 0.25, window, S, H, R, rd, bs,
                                   ws.data_ptr() if nbytes else None, nbytes, None))
    torch.cuda.synchronize()
    for s, n in enumerate(lens):
        rows = torch.stack([cache[int(bt[s, j // bs]) * bs + j % bs] for j in range(n)]).float()
        want = _attention_ref(torch, q_abs[s:s + 1].expand(n, H, R), q_rot[s:s + 1].expand(n, H, rd), rows, window, sink.float(), 0.25)[n - 1]
        assert float((out[s].cpu().double() - want).abs().max()) <= 1e-4, f"sequence {s}"


@pytest.mark.parametrize("window", [7, 64, 256, 257])
def test_window_edge_needle(gpu, window):
    """One key carries a latent far larger than the others and every query points at it: the output jumps between the needle's
    latent (gap = window - 1, still seen) and the background (gap = window, just lost).  The needle sits on a page border."""
    vmx, torch = gpu
    R, rd, H, bs = 16, 4, 1, 8
    T = window + 40
    for needle in (8, 15, 16):                       # first row of a page, last row of a page, next page
        rows = torch.zeros((T, R + rd))
        rows[:, 0] = 0.01
        rows[needle, :R] = 5.0
        rows[needle, R] = 1.0                        # rotated part: only the needle answers the query's rotated part
        q_abs = torch.zeros((T, H, R))
        q_rot = torch.zeros((T, H, rd))
        q_rot[:, :, 0] = 30.0
        got = _attention_op(torch, q_abs, q_rot, rows, window, torch.zeros(H), 1.0, bs, "float32")
        want = _attention_ref(torch, q_abs, q_rot, rows, window, torch.zeros(H), 1.0)
        assert float((got - want).abs().max()) <= 1e-5
        inside, outside = needle + window - 1, needle + window
        assert float(got[inside, 0, 1]) > 4.9 and float(got[outside, 0, 1]) < 1e-3


def test_sink_takes_weight(gpu):
    """A large sink leaves almost nothing for the keys; without it the weights sum to one."""
    vmx, torch = gpu
    T, H, R = 5, 2, 8
    rows = torch.ones((T, R))
    q = torch.zeros((T, H, R))
    with_sink = _attention_op(torch, q, torch.zeros((T, H, 0)), rows, 0, torch.tensor([0.0, 20.0]), 1.0, 4, "float32")
    no_sink = _attention_op(torch, q, torch.zeros((T, H, 0)), rows, 0, None, 1.0, 4, "float32")
    assert np.allclose(no_sink.numpy(), 1.0, atol=1e-6)
    for t in range(T):                               # head 0: sink logit 0 against t + 1 keys of score 0
        assert abs(float(with_sink[t, 0, 0]) - (t + 1) / (t + 2)) < 1e-6
        assert float(with_sink[t, 1, 0]) < 1e-7


# ----------------------------------------------------------------------------- the executor against the oracle

@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_and_layers(gpu, dtype):
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    toks = tokens_for(spec, 45, 1, w)
    logits, _, trace = eng.step([("a", toks, list(range(45)))], layer_trace=True)
    want, layers = orc.forward(spec, w, toks, return_layers=True)
    for i, l in enumerate(layers):
        assert float((trace[i].cpu().double() - l).abs().max()) <= (1e-4 if dtype == "float32" else 0.15) * float(l.abs().max()), f"layer {i}"
    assert rel_err(logits.cpu().numpy(), want.numpy()) <= TOL[dtype]
    model.close()


def test_embedding_alone(gpu):
    """With a zero output projection and no feed-forward the residual stream after the layer is the embedding: scaled token row
    plus hashed bigram row, the extra row for a first token."""
    from tests import gesutar_oracle as orc
    from vllm_rust_amd.gesutar import GesutarLayerSpec
    vmx, torch = gpu
    spec = small_spec(layers=[GesutarLayerSpec(mlp=None, heads=2, dim=8, rot_dim=4, rot_dims=4, vdim=8, kv_rank=16)], bigram_buckets=7,
                      bigram_mul_prev=1000003, bigram_mul_cur=999983, vocab=50021)

    def zero_o(ck):
        ck["l0.mix.o"].zero_()
    model, eng, w = build(spec, "float32", tweak=zero_o)
    toks = [50020, 50020, 3, 50019, 0, 0]            # products beyond 32 bits
    _, _, trace = eng.step([("a", toks, [])], layer_trace=True)
    assert float((trace[0].cpu().double() - orc.embed(toks, w, spec)).abs().max()) <= 1e-5
    model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuttings_agree(gpu, dtype):
    """The same tokens as one prompt, decoded token by token, and in portions of 2, 3, 7 and 16 tokens: every row matches the
    oracle, and in float32 the cuttings match each other to rounding."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    n = 41
    toks = tokens_for(spec, n, 2, w)
    want = orc.forward(spec, w, toks).numpy()
    whole, _, _ = eng.step([("w", toks, list(range(n)))])
    whole = whole.cpu().numpy()
    eng.finish("w")
    assert rel_err(whole, want) <= TOL[dtype]
    for portion in (1, 2, 3, 7, 16):
        got = []
        for a in range(0, n, portion):
            part = toks[a:a + portion]
            lg, _, _ = eng.step([("p", part, list(range(len(part))))])
            got.append(lg.cpu().numpy())
        eng.finish("p")
        got = np.concatenate(got)
        assert rel_err(got, want) <= TOL[dtype], f"portions of {portion}"
        if dtype == "float32":
            assert rel_err(got, whole) <= 2e-5, f"portions of {portion} against the whole prompt"
    model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_unequal_batch_against_each_alone(gpu, dtype):
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    lens = [1, 30, 7, 19]
    full = [tokens_for(spec, n, 10 + i, w, extra=6) for i, n in enumerate(lens)]
    prompts, tails = [f[:n] for f, n in zip(full, lens)], [f[n:] for f, n in zip(full, lens)]
    want = [orc.forward(spec, w, f).numpy() for f in full]
    lg, _, _ = eng.step([(i, p, list(range(len(p)))) for i, p in enumerate(prompts)])
    lg = lg.cpu().numpy()
    at = 0
    for i, p in enumerate(prompts):
        assert rel_err(lg[at:at + len(p)], want[i][:len(p)]) <= TOL[dtype], f"prompt {i} in the batch"
        at += len(p)
    live = [0, 1, 2, 3]
    for s in range(6):                               # decode together; request 2 ends early
        if s == 3:
            eng.finish(2)
            live.remove(2)
        lg, _, _ = eng.step([(i, [tails[i][s]], [0]) for i in live])
        lg = lg.cpu().numpy()
        for j, i in enumerate(live):
            assert rel_err(lg[j:j + 1], want[i][lens[i] + s:lens[i] + s + 1]) <= TOL[dtype], f"request {i}, decoded token {s}"
    model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_batches_on_both_sides_of_the_expert_sort(gpu, dtype):
    """Decode steps of 2, 8 and 12 sequences: up to 16 (token, slot) pairs run their experts unsorted (a pair is its own row
    block), more are sorted into expert blocks; both give the oracle's rows."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, dtype)
    for nseq in (2, 8, 12):
        full = [tokens_for(spec, 3 + i % 4, 60 + i, w, extra=2) for i in range(nseq)]
        want = [orc.forward(spec, w, f).numpy() for f in full]
        eng.step([((nseq, i), f[:-2], []) for i, f in enumerate(full)])
        for s in (2, 1):
            lg, _, _ = eng.step([((nseq, i), [f[-s]], [0]) for i, f in enumerate(full)])
            lg = lg.cpu().numpy()
            for i, f in enumerate(full):
                assert rel_err(lg[i:i + 1], want[i][len(f) - s:len(f) - s + 1]) <= TOL[dtype], f"{nseq} sequences, request {i}"
        for i in range(nseq):
            eng.finish((nseq, i))
    model.close()


def test_blocks_freed_and_used_again(gpu):
    """A second request gets the blocks a finished one gave back (and in another order); two requests that grow in turns own
    interleaved blocks.  Results equal those on an untouched engine."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec()
    model, eng, w = build(spec, "float32", num_blocks=24)
    a, b = tokens_for(spec, 37, 3, w), tokens_for(spec, 29, 4, w)
    eng.step([("a", a, [])])
    used = list(eng.seqs["a"].blocks)
    eng.finish("a")
    lg, _, _ = eng.step([("b", b, list(range(len(b))))])
    assert set(eng.seqs["b"].blocks) <= set(used) and eng.seqs["b"].blocks != used[:len(eng.seqs["b"].blocks)]
    assert rel_err(lg.cpu().numpy(), orc.forward(spec, w, b).numpy()) <= TOL["float32"]
    eng.finish("b")
    got = {"x": [], "y": []}
    for s in range(0, 24, 3):                        # x and y take new blocks alternately
        for name, toks in (("x", a), ("y", b)):
            lg, _, _ = eng.step([(name, toks[s:s + 3], [0, 1, 2])])
            got[name].append(lg.cpu().numpy())
    bx, by = eng.seqs["x"].blocks, eng.seqs["y"].blocks
    assert sorted(bx + by) != bx + by                # the tables are interleaved
    assert rel_err(np.concatenate(got["x"]), orc.forward(spec, w, a[:24]).numpy()) <= TOL["float32"]
    assert rel_err(np.concatenate(got["y"]), orc.forward(spec, w, b[:24]).numpy()) <= TOL["float32"]
    model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sharp_attention_at_window_edges(gpu, dtype):
    """Queries and keys scaled up so that the softmax is nearly one-hot: a key just inside or just outside a window, or on a page
    border, then decides the row.  Windows differ per layer (5 and 12 tokens, pages of 4), prompt then long decoding."""
    from tests import gesutar_oracle as orc
    from vllm_rust_amd.gesutar import GesutarLayerSpec
    vmx, torch = gpu
    base = dict(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=24, rot_dims=8, scale=3.0, experts=4, top=2, groups=1, keep_groups=1,
                expert_ff=16, shared_ff=0)
    spec = small_spec(layers=[GesutarLayerSpec(window=5, **base), GesutarLayerSpec(window=12, **base)])

    def sharpen(ck):
        for i in range(2):
            ck[f"l{i}.mix.sink"].fill_(-4.0)
    model, eng, w = build(spec, dtype, tweak=sharpen)
    n, dec = 30, 40                                   # decoding runs over three windows of the wider layer
    toks = tokens_for(spec, n + dec, 6, w)
    want = orc.forward(spec, w, toks).numpy()
    lg, _, _ = eng.step([("s", toks[:n], list(range(n)))])
    rows = [lg.cpu().numpy()]
    for t in toks[n:]:
        lg, _, _ = eng.step([("s", [t], [0])])
        rows.append(lg.cpu().numpy())
    assert rel_err(np.concatenate(rows), want) <= TOL[dtype] * (1 if dtype == "float32" else 2)
    model.close()


@pytest.mark.parametrize("layer,kw", [
    (dict(heads=1, dim=12, rot_dim=6, rot_dims=4, vdim=10, kv_rank=20, window=1000, experts=5, top=1, groups=1, keep_groups=1, expert_ff=14,
          shared_ff=0), dict(width=40, vocab=61)),
    (dict(heads=5, dim=0, rot_dim=8, rot_dims=8, vdim=8, kv_rank=8, window=1, experts=4, top=4, groups=2, keep_groups=2, expert_ff=8,
          shared_ff=24, router_scale=1.0), dict(width=24, bigram_buckets=1)),
    (dict(heads=2, dim=16, rot_dim=0, rot_dims=0, vdim=12, kv_rank=72, window=3, mlp=None), dict(width=56)),
])
def test_other_sizes(gpu, layer, kw):
    """Sizes that are not multiples of 8, one head, no unrotated or no rotated dimensions, partly rotated vectors, a window of one
    token and one longer than the sequence, top = experts, a single group, no shared expert, a layer without feed-forward."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = small_spec(layer=layer, **kw)
    for dtype in ("float32", "bfloat16"):
        model, eng, w = build(spec, dtype, seed=3)
        toks = tokens_for(spec, 23, 7, w)
        want = orc.forward(spec, w, toks).numpy()
        lg, _, _ = eng.step([("a", toks[:17], list(range(17)))])
        rows = [lg.cpu().numpy()]
        for t in toks[17:]:
            lg, _, _ = eng.step([("a", [t], [0])])
            rows.append(lg.cpu().numpy())
        assert rel_err(np.concatenate(rows), want) <= TOL[dtype]
        model.close()


def test_greedy_generation_through_the_scheduler(gpu):
    """Engine.generate: more requests than fit at once, prompts fed in portions, greedy ids from the library's argmax; the ids
    equal the oracle's greedy continuation of each prompt alone."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    from vllm_rust_amd.engine import SamplingParams
    spec = small_spec()
    model, eng, w = build(spec, "float32", num_blocks=20, block_size=4)      # 80 cache rows: the five requests cannot all be live
    prompts = [tokens_for(spec, n, 30 + i) for i, n in enumerate([9, 21, 3, 14, 1])]
    out = eng.generate(prompts, SamplingParams(max_new_tokens=8), prefill_chunk=5)
    for p, o in zip(prompts, out):
        assert o == orc.greedy(spec, w, p, 8)
    assert len(eng.blocks.free) == 20 and not eng.seqs
    model.close()


def test_sampling_through_the_engine(gpu):
    """Temperature sampling with top-k 1 is greedy, whatever the draw."""
    vmx, torch = gpu
    from vllm_rust_amd.engine import SamplingParams
    spec = small_spec()
    model, eng, w = build(spec, "float32")
    prompts = [tokens_for(spec, 6, 40), tokens_for(spec, 11, 41)]
    greedy = eng.generate(prompts, SamplingParams(max_new_tokens=5))
    drawn = eng.generate(prompts, SamplingParams(max_new_tokens=5, temperature=0.8, top_k=1, seed=3))
    assert greedy == drawn
    model.close()


def test_checkpoint_directory_and_registry(gpu, tmp_path):
    """config.json + model.safetensors written from a spec load back through the registry and give the same logits."""
    import json
    from safetensors.torch import save_file
    vmx, torch = gpu
    from vllm_rust_amd.engine import Engine
    from vllm_rust_amd.gesutar import GesutarSpec, synthetic_weights
    from vllm_rust_amd.models import load_model
    spec = small_spec()
    ck = synthetic_weights(spec, 9)
    (tmp_path / "config.json").write_text(json.dumps(spec.to_config()))
    save_file(ck, str(tmp_path / "model.safetensors"))
    assert GesutarSpec.from_config(spec.to_config()) == spec
    model = load_model(tmp_path, dtype="bfloat16", max_tokens=64, max_seqs=4, block_size=8)
    m2, eng2, _ = build(spec, "bfloat16", seed=9)
    toks = tokens_for(spec, 12, 8)
    a, _, _ = Engine(model).step([(0, toks, [11])])
    b, _, _ = eng2.step([(0, toks, [11])])
    assert torch.equal(a, b)
    model.close()
    m2.close()


def test_trace_replay_tool(gpu, tmp_path):
    """bin/trace_run on a checkpoint directory: two requests start together, one goes on alone; the files hold the oracle's rows."""
    import json
    import subprocess
    import sys
    from pathlib import Path
    from safetensors.torch import save_file
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    from vllm_rust_amd.gesutar import synthetic_weights
    spec = small_spec()
    ck = synthetic_weights(spec, 11)
    (tmp_path / "m").mkdir()
    (tmp_path / "m" / "config.json").write_text(json.dumps(spec.to_config()))
    save_file(ck, str(tmp_path / "m" / "model.safetensors"))
    w = {k: v.double() for k, v in ck.items()}
    a, b = tokens_for(spec, 9, 50, w), tokens_for(spec, 4, 51, w)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}, {"id": "b", "tokens": b, "want": [3]}], "end": ["b"]},
             {"step": 1, "entries": [{"id": "a", "tokens": a[7:8], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": a[8:9], "want": [0]}], "end": ["a"]}]
    root = Path(__file__).resolve().parent.parent
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / dtype
        r = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(tmp_path / "m"), "--dtype", dtype, "--out", str(out),
                            "--max-tokens", "64"], input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr[-2000:]
        assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
        wa, wb = orc.forward(spec, w, a).numpy(), orc.forward(spec, w, b).numpy()
        s0 = np.fromfile(out / "0.f32", dtype="<f4").reshape(3, spec.vocab)
        s2 = np.fromfile(out / "2.f32", dtype="<f4").reshape(1, spec.vocab)
        assert not (out / "1.f32").exists()
        assert rel_err(s0, np.stack([wa[0], wa[6], wb[3]])) <= TOL[dtype] and rel_err(s2, wa[8:9]) <= TOL[dtype]


def test_engine_serves_the_qwen3_executor_too(gpu):
    """The same Engine (block manager, scheduler, packed steps) over the Qwen3 executor through its adapter: greedy ids of three
    prompts generated together equal each prompt generated alone on an untouched engine."""
    vmx, torch = gpu
    from vllm_rust_amd.engine import Engine, PackedQwen3, SamplingParams
    from vllm_rust_amd.qwen3 import QuantizedQwen3ForCausalLM, Qwen3Spec
    spec = Qwen3Spec(hidden_size=256, num_layers=2, num_heads=4, num_kv_heads=2, head_dim=64, intermediate_size=512, vocab_size=1000,
                     max_position=256, num_blocks=24, max_batch=4, max_seq_len=128, max_prefill_tokens=64)
    model = QuantizedQwen3ForCausalLM(spec)
    model.load_synthetic(seed=2)
    prompts = [np.random.default_rng(70 + i).integers(0, 1000, n).tolist() for i, n in enumerate([5, 17, 1])]
    together = Engine(PackedQwen3(model)).generate(prompts, SamplingParams(max_new_tokens=6))
    alone = [Engine(PackedQwen3(model)).generate([p], SamplingParams(max_new_tokens=6))[0] for p in prompts]
    assert together == alone and all(len(o) == 6 for o in together)
    model.close()


def _random_spec(seed):
    """A configuration drawn at random: per-layer sizes, windows, rotation, router shape; some layers without feed-forward."""
    from vllm_rust_amd.gesutar import GesutarLayerSpec, GesutarSpec
    r = np.random.default_rng(seed)
    pick = lambda *xs: xs[int(r.integers(0, len(xs)))]
    step = pick(8, 8, 2)                                      # multiples of 8 take the matrix-core attention, others the vector form
    layers = []
    for li in range(int(r.integers(1, 4))):
        dim, rd = pick((0, 2), (1, 1), (2, 1), (3, 2), (1, 0), (5, 3))
        dim, rd = dim * step, rd * step
        rot_dims = 0 if rd == 0 else pick(rd, rd, max(2, rd // 2 // 2 * 2))
        groups = pick(1, 2, 3)
        per = pick(1, 2, 4)
        keep = int(r.integers(1, groups + 1))
        moe = li == 0 or r.random() < 0.7
        layers.append(GesutarLayerSpec(heads=int(r.integers(1, 10)), dim=dim, rot_dim=rd, vdim=pick(1, 3, 5) * step, kv_rank=pick(1, 2, 5, 9, 17) * step,
                                       window=pick(1, 2, 7, 16, 33, 65, 500), rot_dims=rot_dims, rot_base=pick(100.0, 10000.0, 5e5),
                                       scale=pick(0.1, 0.25, 0.5), mlp="moe" if moe else None, experts=groups * per,
                                       top=int(r.integers(1, keep * per + 1)), groups=groups, keep_groups=keep, expert_ff=pick(6, 16, 40),
                                       shared_ff=pick(0, 8, 24), router_scale=pick(1.0, 2.5)))
    return GesutarSpec(vocab=pick(17, 100, 257), width=pick(24, 40, 64, 72), layers=layers, norm_eps=pick(1e-5, 1e-6), embed_scale=pick(1.0, 4.0),
                       bigram_buckets=pick(1, 31, 509), bigram_mul_prev=pick(1, 31, 65537), bigram_mul_cur=pick(1, 7))


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(gpu, seed):
    """Ten configurations drawn at random, each a 45-token prompt and 25 decoded tokens in both modes against the oracle."""
    from tests import gesutar_oracle as orc
    vmx, torch = gpu
    spec = _random_spec(seed)
    for dtype in ("float32", "bfloat16"):
        model, eng, w = build(spec, dtype, seed=seed, block_size=int(np.random.default_rng(seed).integers(1, 9)), num_blocks=96)
        toks = tokens_for(spec, 70, 100 + seed, w if dtype == "bfloat16" else None)
        want = orc.forward(spec, w, toks).numpy()
        lg, _, _ = eng.step([("r", toks[:45], list(range(45)))])
        rows = [lg.cpu().numpy()]
        for t in toks[45:]:
            lg, _, _ = eng.step([("r", [t], [0])])
            rows.append(lg.cpu().numpy())
        assert rel_err(np.concatenate(rows), want) <= TOL[dtype] * (1 if dtype == "float32" else 1.5), f"{dtype}: {spec}"
        model.close()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windows_over_several_key_tiles(gpu, dtype):
    """A 230-token prompt and 40 decoded tokens through layers whose windows (150 and 70 tokens) span several 64-key tiles of the
    matrix-core attention, so that prompts walk many tiles and decode steps split their keys over partitions; far keys matter
    because the sinks are low and the scores sharp."""
    from tests import gesutar_oracle as orc
    from vllm_rust_amd.gesutar import GesutarLayerSpec
    vmx, torch = gpu
    base = dict(heads=4, dim=16, rot_dim=8, vdim=16, kv_rank=32, rot_dims=8, scale=1.5, experts=2, top=2, groups=1, keep_groups=1,
                expert_ff=16, shared_ff=8)      # every expert is chosen: no router decision that rounding could flip
    spec = small_spec(layers=[GesutarLayerSpec(window=150, **base), GesutarLayerSpec(window=70, **base)])

    def low_sinks(ck):
        for i in range(2):
            ck[f"l{i}.mix.sink"].fill_(-6.0)
    model, eng, w = build(spec, dtype, tweak=low_sinks, block_size=16, num_blocks=40, max_tokens=512)
    toks = tokens_for(spec, 270, 9, w if dtype == "bfloat16" else None)
    want = orc.forward(spec, w, toks).numpy()
    lg, _, _ = eng.step([("s", toks[:230], list(range(230)))])
    rows = [lg.cpu().numpy()]
    for t in toks[230:]:
        lg, _, _ = eng.step([("s", [t], [0])])
        rows.append(lg.cpu().numpy())
    assert rel_err(np.concatenate(rows), want) <= TOL[dtype] * (1 if dtype == "float32" else 1.5)
    model.close()
