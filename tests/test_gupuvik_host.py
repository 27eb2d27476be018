"""Host-side parts of serving Gupuvik, without a GPU: configuration reading (ranks from tensor shapes), the registry, the
oracle's own mechanisms on hand-made inputs, the state-slot manager, and the step function / scheduler driven by a stand-in model
with recurrent state."""
import json
import math

import numpy as np
import pytest
import torch

from tests import gupuvik_oracle as orc


def _spec():
    from vllm_rust_amd.gupuvik import GupuvikLayerSpec, GupuvikSpec
    layers = [GupuvikLayerSpec(mixer="channel_delta", heads=4, kv_heads=2, dim=6, vdim=10, conv=3, decay_rank=5, gate_rank=7, mlp="dense", ff=20),
              GupuvikLayerSpec(mixer="attention", heads=4, kv_heads=1, dim=6, vdim=4, window=9, keep_first=2, scale=0.4, softcap=11.0, mlp="moe",
                               experts=3, top=2, expert_ff=8),
              GupuvikLayerSpec(mixer="attention", heads=4, kv_heads=1, dim=6, vdim=4, window=3, kv_from=1, mlp=None)]
    return GupuvikSpec(vocab=31, width=16, layers=layers, norm_eps=1e-5, embed_scale=1.5)


def test_config_round_trip_and_sizes_from_tensor_shapes():
    from vllm_rust_amd.gupuvik import GupuvikLayerSpec, GupuvikSpec
    spec = _spec()
    cfg = spec.to_config()
    shapes = spec.tensor_shapes()
    assert "decay_rank" not in json.dumps(cfg)                  # the configuration states no ranks ...
    assert GupuvikSpec.from_config(cfg, shapes) == spec         # ... the shapes of a1 / g1 do
    assert cfg["architecture"] == "Gupuvik" and cfg["layers"][2]["mlp"] is None and cfg["layers"][2]["mixer"]["kv_from"] == 1
    names = list(shapes)
    assert names[0] == "embed" and names[-1] == "head" and shapes["l0.norm1"] == () and shapes["final.norm"] == ()
    assert "l2.mix.k" not in shapes and "l2.rg2" not in shapes and shapes["l1.mix.k"] == (6, 16) and shapes["l0.mix.a2"] == (24, 5)
    assert shapes["l0.mix.q.conv"] == (12, 3) and shapes["l0.mix.b"] == (4, 16) and shapes["l1.mlp.e2.gate"] == (8, 16)
    # absent mask / cap / kv_heads: no window, no cap, as many key heads as query heads
    l = GupuvikLayerSpec.from_config({"type": "attention", "mixer": {"heads": 2, "dim": 8, "vdim": 4, "scale": 0.5}, "mlp": None})
    assert (l.window, l.keep_first, l.softcap, l.kv_heads, l.kv_from, l.mlp) == (0, 0, 0.0, 2, None, None)
    with pytest.raises(ValueError):
        GupuvikLayerSpec.from_config({"type": "something_else", "mixer": {}})
    with pytest.raises(ValueError):
        GupuvikLayerSpec.from_config({"type": "attention", "mixer": {"heads": 2, "dim": 8}, "mlp": {"kind": "other"}})


def test_registry_knows_the_architecture(tmp_path):
    from vllm_rust_amd import models
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Gupuvik"}))
    assert models.architecture_of(tmp_path) == "Gupuvik" and "Gupuvik" in models.REGISTRY and "Gesutar" in models.REGISTRY


def test_oracle_visibility():
    see = [[j for j in range(12) if orc.visible(i, j, 3, 2)] for i in range(12)]
    assert see[0] == [0] and see[2] == [0, 1, 2] and see[4] == [0, 1, 2, 3, 4] and see[5] == [0, 1, 3, 4, 5] and see[11] == [0, 1, 9, 10, 11]
    assert [j for j in range(6) if orc.visible(5, j, 1, 0)] == [5]


def test_oracle_convolution_and_units():
    x = torch.tensor([[1.0, 2.0], [0.0, 1.0], [3.0, 0.0]], dtype=torch.float64)
    taps = torch.tensor([[10.0, 1.0], [0.5, 2.0]], dtype=torch.float64)       # last column multiplies the current token
    pre = torch.tensor([[1.0, 4.0], [10.0, 3.0], [3.0, 0.5]], dtype=torch.float64)
    assert torch.allclose(orc.causal_conv_silu(x, taps), pre * torch.sigmoid(pre))
    u = orc.unit(torch.tensor([[3.0, 4.0]], dtype=torch.float64))
    assert abs(float((u * u).sum()) - 25 / (25 + 1e-6)) < 1e-12
    assert abs(float(orc.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


def test_oracle_delta_rule_overwrites_a_key():
    """With unit keys, beta = 1 and no decay the memory returns exactly the last value written under a key; a decay of g on the
    key's channel leaves g of the old value to be corrected."""
    k = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]], [[1.0, 0.0]]], dtype=torch.float64)
    v = torch.tensor([[[5.0]], [[7.0]], [[9.0]]], dtype=torch.float64)
    one = torch.ones((3, 1), dtype=torch.float64)
    o = orc.delta_rule_scan(k, k, v, one, torch.ones((3, 1, 2), dtype=torch.float64))
    assert o.flatten().tolist() == [5.0, 7.0, 9.0]
    half = torch.full((3, 1), 0.5, dtype=torch.float64)
    o = orc.delta_rule_scan(k, k, v, half, torch.full((3, 1, 2), 0.5, dtype=torch.float64))
    # t0: S = 2.5 under key 0; halved at t1 and again at t2: 0.625; u = 0.5 (9 - 0.625), read-out 0.625 + 4.1875
    assert np.allclose(o.flatten().numpy(), [2.5, 3.5, 4.8125])


def test_oracle_router_and_layer_are_consistent():
    z = torch.tensor([[1.0, 3.0, 2.0, -1.0]], dtype=torch.float64)
    idx, wt, _ = orc.route(torch.eye(4, dtype=torch.float64)[:1] * 0 + 1, {"router": z.T.repeat(1, 4) / 4}, "", 2)
    e = math.exp(-1.0)
    assert idx.tolist() == [[1, 2]] and np.allclose(wt.numpy(), [[1 / (1 + e), e / (1 + e)]])
    from vllm_rust_amd.gupuvik import synthetic_weights
    spec = _spec()
    w = {k: v.double() for k, v in synthetic_weights(spec, 0).items()}
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7]
    full, layers = orc.forward(toks, w, spec.to_config(), return_layers=True)
    assert layers.shape == (3, 14, 16) and torch.allclose(orc.forward(toks[:9], w, spec.to_config()), full[:9])   # causal


def test_state_slots_are_handed_out_again():
    from vllm_rust_amd.engine import StateSlots
    s = StateSlots(3)
    a, b, c = s.allocate(), s.allocate(), s.allocate()
    assert (a, b, c) == (0, 1, 2)
    with pytest.raises(MemoryError):
        s.allocate()
    s.release(b)
    s.release(a)
    assert s.allocate() == a and s.allocate() == b


class _Recurrent:
    """Stand-in model with recurrent state: records what each step was given; greedy id = (token + position) mod vocab."""
    block_size, num_blocks, max_tokens, max_seqs, vocab_size, state_slots, device = 4, 12, 16, 2, 50, 2, torch.device("cpu")

    def __init__(self):
        self.steps = []

    def forward(self, tokens, prev, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits=True, want_greedy=False,
                layer_trace=False, seq_starts=None, state_slots=None):
        self.steps.append(dict(tokens=tokens.tolist(), pos=positions.tolist(), starts=seq_starts.tolist(), state=state_slots.tolist()))
        if logit_rows is None:
            return None, None, None
        ids = ((tokens + positions) % self.vocab_size)[logit_rows.long()].to(torch.int32)
        return (torch.nn.functional.one_hot(ids.long(), self.vocab_size).float() if want_logits else None), (ids if want_greedy else None), None


def test_step_hands_every_sequence_its_rows_and_state_slot():
    from vllm_rust_amd.engine import Engine
    m = _Recurrent()
    eng = Engine(m)
    eng.step([("a", [7, 8, 9], [2]), ("b", [5], [])])
    eng.step([("b", [6], [0]), ("a", [3], [0])])
    assert m.steps[0]["starts"] == [0, 3, 4] and m.steps[0]["state"] == [0, 1]
    assert m.steps[1]["starts"] == [0, 1, 2] and m.steps[1]["state"] == [1, 0] and m.steps[1]["pos"] == [1, 3]
    with pytest.raises(MemoryError):
        eng.step([("c", [1], [])])
    eng.finish("a")
    eng.step([("c", [1, 2], [])])
    assert m.steps[-1]["state"] == [0] and m.steps[-1]["pos"] == [0, 1]      # a's slot, from position 0: the executor starts it empty


def test_scheduler_never_runs_more_sequences_than_state_slots():
    from vllm_rust_amd.engine import Engine, SamplingParams
    m = _Recurrent()
    eng = Engine(m)
    out = eng.generate([[1] * 5, [2] * 7, [3] * 2], SamplingParams(max_new_tokens=3), prefill_chunk=4)
    assert [len(o) for o in out] == [3, 3, 3] and max(len(s["state"]) for s in m.steps) <= 2
    assert not eng.seqs and sorted(eng.states.free) == [0, 1] and len(eng.blocks.free) == 12
