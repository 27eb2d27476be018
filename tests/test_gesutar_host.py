"""Host-side parts of serving Gesutar, without a GPU: configuration reading, the oracle's own mechanisms on hand-made inputs, the
block manager, and the scheduler driven by a stand-in model."""
import math

import numpy as np
import pytest
import torch

from tests import gesutar_oracle as orc


def test_config_round_trip_and_defaults():
    from vllm_rust_amd.gesutar import GesutarLayerSpec, GesutarSpec
    spec = GesutarSpec(vocab=70, width=32, layers=[GesutarLayerSpec(), GesutarLayerSpec(mlp=None, window=5)], embed_scale=2.0,
                       bigram_buckets=11, bigram_mul_prev=3, bigram_mul_cur=2)
    cfg = spec.to_config()
    assert GesutarSpec.from_config(cfg) == spec
    assert cfg["layers"][1]["mlp"] is None and cfg["layers"][1]["mixer"]["mask"]["size"] == 5
    # absent groups / shared expert / rotation: one group, no shared expert, the whole rotated part rotates
    entry = {"type": "latent_attention", "mixer": {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 8, "kv_rank": 16, "mask": {"size": 9}, "scale": 0.5},
             "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 4, "top": 2}}}
    l = GesutarLayerSpec.from_config(entry)
    assert (l.groups, l.keep_groups, l.shared_ff, l.rot_dims, l.router_scale) == (1, 1, 0, 4, 1.0)
    with pytest.raises(ValueError):
        GesutarLayerSpec.from_config(dict(entry, type="something_else"))
    names = list(spec.tensor_shapes())
    assert names[0] == "embed" and names[-1] == "head" and "l1.norm2" not in names and "l0.mlp.e7.down" in names


def test_registry_picks_the_class_by_config(tmp_path):
    import json
    from vllm_rust_amd import models
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Gesutar"}))
    assert models.architecture_of(tmp_path) == "Gesutar" and "Gesutar" in models.REGISTRY
    (tmp_path / "config.json").write_text(json.dumps({"architectures": ["NoSuchModel"]}))
    with pytest.raises(NotImplementedError):
        models.load_model(tmp_path)


def test_oracle_bigram_rows():
    assert orc.hashed_bigram_rows([3, 4, 4], -1, 7, 10, 1) == [7, (3 * 10 + 4) % 7, (4 * 10 + 4) % 7]
    assert orc.hashed_bigram_rows([5], 2, 7, 10, 1) == [(2 * 10 + 5) % 7]


def test_oracle_rotation_is_a_rotation_of_pairs():
    x = torch.tensor([[1.0, 0.0, 0.0, 2.0, 9.0]], dtype=torch.float64)
    y = orc.rotate_pairs(x, torch.tensor([1]), 4, 100.0)
    a0, a1 = 1.0, 100.0 ** -0.5
    want = [math.cos(a0), math.sin(a0), -2 * math.sin(a1), 2 * math.cos(a1), 9.0]
    assert np.allclose(y.numpy()[0], want) and np.allclose(orc.rotate_pairs(x, torch.tensor([0]), 4, 100.0).numpy(), x.numpy())


def test_oracle_sink_and_window():
    sc = torch.zeros((1, 3), dtype=torch.float64)
    p = orc.softmax_with_sink(sc, torch.tensor([[True, True, False]]), torch.tensor(0.0, dtype=torch.float64))
    assert np.allclose(p.numpy(), [[1 / 3, 1 / 3, 0.0]])
    p = orc.softmax_with_sink(sc, torch.tensor([[True, True, False]]), None)
    assert np.allclose(p.numpy(), [[0.5, 0.5, 0.0]])


def test_oracle_router_groups():
    z = torch.log(torch.tensor([[0.30, 0.05, 0.25, 0.24, 0.10, 0.06]]))
    # groups of two: scores 0.30, 0.25, 0.10 -> groups 0 and 1 kept; top 3 among experts 0..3
    ids, w = orc.grouped_router(z, 6, 3, 2, 3, 2.0)
    assert ids == [[0, 2, 3]] and np.allclose(w.numpy(), 2.0 * np.array([[0.30, 0.25, 0.24]]) / 0.79)
    ids, _ = orc.grouped_router(z, 6, 3, 1, 2, 1.0)
    assert ids == [[0, 1]]                       # the second-best expert overall (2) lies outside the kept group


def test_block_manager_reuses_freed_blocks():
    from vllm_rust_amd.engine import BlockManager
    bm = BlockManager(6, 4)
    a = bm.allocate(bm.blocks_for(9))
    assert a == [0, 1, 2] and bm.blocks_for(8) == 2 and bm.blocks_for(1) == 1
    b = bm.allocate(2)
    bm.release(a)
    assert bm.allocate(2) == [2, 1] and bm.can_allocate(2) and not bm.can_allocate(3)
    with pytest.raises(MemoryError):
        bm.allocate(3)
    bm.release(b)


class _Echo:
    """Stand-in model: the greedy id of a row is (token + position) mod vocab; records what each step was given."""
    block_size, num_blocks, max_tokens, max_seqs, vocab_size, device = 4, 12, 16, 3, 50, torch.device("cpu")

    def __init__(self):
        self.steps = []

    def forward(self, tokens, prev, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits=True, want_greedy=False,
                layer_trace=False):
        self.steps.append(dict(tokens=tokens.tolist(), prev=prev.tolist(), pos=positions.tolist(), slots=slots.tolist(), sid=seq_ids.tolist(),
                               bt=block_tables.tolist()))
        if logit_rows is None:
            return None, None, None
        rows = logit_rows.long()
        ids = ((tokens + positions) % self.vocab_size)[rows].to(torch.int32)
        logits = torch.nn.functional.one_hot(ids.long(), self.vocab_size).float()
        return (logits if want_logits else None), (ids if want_greedy else None), None


def test_step_builds_positions_slots_and_previous_tokens():
    from vllm_rust_amd.engine import Engine
    m = _Echo()
    eng = Engine(m)
    eng.step([("a", [7, 8, 9, 1, 2], [4]), ("b", [5], [])])
    eng.step([("b", [6], [0]), ("a", [3], [0])])
    s0, s1 = m.steps
    assert s0["prev"] == [-1, 7, 8, 9, 1, -1] and s0["pos"] == [0, 1, 2, 3, 4, 0] and s0["sid"] == [0, 0, 0, 0, 0, 1]
    assert s0["bt"] == [[0, 1], [2, 0]] and s0["slots"] == [0, 1, 2, 3, 4, 8]
    assert s1["prev"] == [5, 2] and s1["pos"] == [1, 5] and s1["slots"] == [9, 5] and s1["bt"] == [[2, 0], [0, 1]]
    eng.finish("a")
    eng.step([("c", [1] * 9, [])])
    assert eng.seqs["c"].blocks == [1, 0, 3]     # a's blocks first, then a fresh one
    with pytest.raises(ValueError):
        eng.step([("d", [0] * 17, [])])


def test_scheduler_feeds_portions_and_admits_when_blocks_free_up():
    from vllm_rust_amd.engine import Engine, SamplingParams
    m = _Echo()
    eng = Engine(m)
    prompts = [[1] * 10, [2] * 13, [3] * 2, [4] * 6]
    out = eng.generate(prompts, SamplingParams(max_new_tokens=4), prefill_chunk=6)

    def expect(p):
        seq, o = list(p), []
        for _ in range(4):
            o.append((seq[-1] + len(seq) - 1) % 50)
            seq.append(o[-1])
        return o
    assert out == [expect(p) for p in prompts]
    assert max(len(s["tokens"]) for s in m.steps) <= 16 and max(len(s["bt"]) for s in m.steps) <= 3
    assert any(len(set(s["sid"])) > 1 and len(s["tokens"]) == len(set(s["sid"])) for s in m.steps)      # a joint decode step happened
    assert not eng.seqs and len(eng.blocks.free) == 12
