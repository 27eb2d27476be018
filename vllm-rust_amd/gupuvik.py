"""Host-side driver of the Gupuvik decoder family (libvmx `vmx_gupuvik_*`).

A Gupuvik model is a stack of parallel layers listed in its config.json: one scalar-gain RMS norm feeds a token mixer and an
optional feed-forward, and each sublayer's result enters the residual stream through an element-wise sigmoid gate.  Mixers:
"attention" (grouped-query, biased projections, no rotation, per-head temperature, tanh soft cap, sliding window that keeps the
first tokens, per-head output gate, optionally reading an earlier layer's key/value cache) and "channel_delta" (short causal
convolutions, gated delta rule with per-channel decay; its state lives in a per-sequence state slot).  Feed-forward: "dense"
(tanh GELU) or "moe" (SiLU-gated experts, softmax over the chosen router logits).  This file reads the configuration (sizes the
configuration does not state, the ranks of the low-rank projections, come from the tensors' shapes), hands the checkpoint's
tensors to the library under their file names and wraps the one forward entry point.  All arithmetic happens in the library.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import json
import math
import re
from pathlib import Path

import numpy as np
import torch

from ._lib import GupuvikConfig, GupuvikLayerConfig, check, lib

VMX_F32, VMX_BF16 = 0, 1
MIXERS = {"attention": 1, "channel_delta": 2}
MLPS = {None: 0, "dense": 2, "moe": 3}


@dataclasses.dataclass
class GupuvikLayerSpec:
    mixer: str = "attention"
    heads: int = 4
    kv_heads: int = 2
    dim: int = 32
    vdim: int = 32
    # attention
    window: int = 0              # 0: every earlier key
    keep_first: int = 0
    scale: float = 0.125
    softcap: float = 0.0         # 0: none
    kv_from: int | None = None
    # channel delta
    conv: int = 4
    decay_rank: int = 8
    gate_rank: int = 8
    # feed-forward
    mlp: str | None = "dense"
    ff: int = 64
    experts: int = 0
    top: int = 0
    expert_ff: int = 0

    @staticmethod
    def from_config(entry: dict, ranks: dict | None = None) -> "GupuvikLayerSpec":
        """ranks: {"decay": r, "gate": r} of a channel_delta layer, read from the shapes of its a1 / g1 tensors."""
        kind = entry["type"]
        if kind not in MIXERS:
            raise ValueError(f"Gupuvik: unknown layer type `{kind}`")
        m = entry["mixer"]
        s = GupuvikLayerSpec(mixer=kind, heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                             vdim=int(m.get("vdim", m["dim"])), mlp=None)
        if kind == "attention":
            mask = m.get("mask") or {}
            s.window, s.keep_first = int(mask.get("size", 0)), int(mask.get("keep_first", 0))
            s.scale = float(m.get("scale", 1.0 / math.sqrt(s.dim)))
            s.softcap = float(m.get("softcap") or 0.0)
            s.kv_from = None if m.get("kv_from") is None else int(m["kv_from"])
        else:
            s.conv = int(m["conv"])
            ranks = ranks or {}
            s.decay_rank, s.gate_rank = int(ranks.get("decay", m.get("decay_rank", 0))), int(ranks.get("gate", m.get("gate_rank", 0)))
        ff = entry.get("mlp")
        if ff is not None:
            s.mlp = ff["kind"]
            if s.mlp == "dense":
                s.ff = int(ff["ff"])
            elif s.mlp == "moe":
                s.experts, s.top, s.expert_ff = int(ff["router"]["experts"]), int(ff["router"]["top"]), int(ff["expert"]["ff"])
            else:
                raise ValueError(f"Gupuvik: unknown feed-forward kind `{s.mlp}`")
        return s

    def to_config(self) -> dict:
        if self.mixer == "attention":
            m = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
            if self.softcap:
                m["softcap"] = self.softcap
            if self.window:                  # no window: every earlier key is visible and there is no mask to state
                m["mask"] = {"size": self.window, "keep_first": self.keep_first}
            if self.kv_from is not None:
                m["kv_from"] = self.kv_from
        else:
            m = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        ff = None
        if self.mlp == "dense":
            ff = {"kind": "dense", "ff": self.ff}
        elif self.mlp == "moe":
            ff = {"kind": "moe", "expert": {"ff": self.expert_ff}, "router": {"experts": self.experts, "top": self.top}}
        return {"type": self.mixer, "mixer": m, "mlp": ff}


@dataclasses.dataclass
class GupuvikSpec:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    embed_scale: float = 1.0

    @staticmethod
    def from_config(cfg: dict, shapes: dict | None = None) -> "GupuvikSpec":
        """shapes: name -> shape of the checkpoint's tensors (for the sizes the configuration leaves to them)."""
        layers = []
        for i, e in enumerate(cfg["layers"]):
            ranks = None
            if shapes is not None and e["type"] == "channel_delta":
                ranks = {"decay": shapes[f"l{i}.mix.a1"][0], "gate": shapes[f"l{i}.mix.g1"][0]}
            layers.append(GupuvikLayerSpec.from_config(e, ranks))
        return GupuvikSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=layers, norm_eps=float(cfg["norm"]["eps"]),
                           embed_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)))

    def to_config(self) -> dict:
        return {"architecture": "Gupuvik", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embed_scale}, "layers": [l.to_config() for l in self.layers]}

    @property
    def recurrent(self) -> bool:
        return any(l.mixer == "channel_delta" for l in self.layers)

    def tensor_shapes(self) -> dict:
        """Name -> shape of every checkpoint tensor, in file order."""
        W, out = self.width, {}
        out["embed"] = (self.vocab, W)
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = ()
            if l.mixer == "attention":
                out[p + "mix.q"], out[p + "mix.q.b"] = (l.heads * l.dim, W), (l.heads * l.dim,)
                if l.kv_from is None:
                    out[p + "mix.k"], out[p + "mix.k.b"] = (l.kv_heads * l.dim, W), (l.kv_heads * l.dim,)
                    out[p + "mix.v"], out[p + "mix.v.b"] = (l.kv_heads * l.vdim, W), (l.kv_heads * l.vdim,)
                out[p + "mix.temp"] = (l.heads,)
                out[p + "mix.g"] = (l.heads, W)
                out[p + "mix.o"] = (W, l.heads * l.vdim)
            else:
                for n, c in (("q", l.kv_heads * l.dim), ("k", l.kv_heads * l.dim), ("v", l.heads * l.vdim)):
                    out[p + "mix." + n] = (c, W)
                    out[p + f"mix.{n}.conv"] = (c, l.conv)
                out[p + "mix.b"] = (l.heads, W)
                out[p + "mix.A_log"] = (l.heads,)
                out[p + "mix.norm"] = (l.vdim,)
                out[p + "mix.a1"], out[p + "mix.a2"] = (l.decay_rank, W), (l.heads * l.dim, l.decay_rank)
                out[p + "mix.dt_bias"] = (l.heads * l.dim,)
                out[p + "mix.g1"], out[p + "mix.g2"] = (l.gate_rank, W), (l.heads * l.vdim, l.gate_rank)
                out[p + "mix.o"] = (W, l.heads * l.vdim)
            if l.mlp == "dense":
                out[p + "mlp.up"], out[p + "mlp.down"] = (l.ff, W), (W, l.ff)
            elif l.mlp == "moe":
                for e in range(l.experts):
                    out[p + f"mlp.e{e}.gate"] = (l.expert_ff, W)
                    out[p + f"mlp.e{e}.up"] = (l.expert_ff, W)
                    out[p + f"mlp.e{e}.down"] = (W, l.expert_ff)
                out[p + "mlp.router"] = (l.experts, W)
            out[p + "rg1"], out[p + "rg1.b"] = (W, W), (W,)
            if l.mlp:
                out[p + "rg2"], out[p + "rg2.b"] = (W, W), (W,)
        out["final.norm"] = ()
        out["head"] = (self.vocab, W)
        return out


def synthetic_weights(spec: GupuvikSpec, seed: int = 0, device="cpu") -> dict:
    """Seeded random-init checkpoint (bf16 tensors on `device`): matrices ~ 1 / sqrt(in), gains around 1, temperatures around 1,
    decay rates and step biases such that memories fade over tens of tokens; activations stay O(1) through the stack."""
    g = torch.Generator(device=device).manual_seed(seed)

    def randn(shape):
        return torch.randn(shape, generator=g, device=device)
    ck = {}
    for name, shape in spec.tensor_shapes().items():
        if name.endswith("norm1") or name == "final.norm" or name.endswith("mix.norm") or name.endswith("mix.temp"):
            t = 1.0 + 0.1 * randn(shape)
        elif name.endswith("A_log"):
            t = -1.0 + 0.5 * randn(shape)
        elif name.endswith("dt_bias"):
            t = -1.0 + 0.5 * randn(shape)
        elif name.endswith(".b") and not name.endswith("mix.b"):
            t = 0.2 * randn(shape)
        elif name.endswith(".conv"):
            t = randn(shape) / math.sqrt(shape[-1])
        elif name == "embed":
            t = randn(shape) / max(spec.embed_scale, 1e-6)
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        ck[name] = t.to(torch.bfloat16)
    return ck


class GupuvikForCausalLM:
    """The executor handle: weights, paged key/value caches, recurrent-state slots and workspaces live in the library."""

    architecture = "Gupuvik"

    def __init__(self, spec: GupuvikSpec, dtype: str = "bfloat16", block_size: int = 16, num_blocks: int = 256, max_tokens: int = 2048,
                 max_seqs: int = 64, device: int = 0):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"Gupuvik runs in bfloat16 or float32, not `{dtype}`")
        self.spec, self.dtype = spec, dtype
        self.block_size, self.num_blocks, self.max_tokens, self.max_seqs = block_size, num_blocks, max_tokens, max_seqs
        self.vocab_size = spec.vocab
        self.state_slots = max_seqs          # the engine hands one to every live sequence
        self.device = torch.device("cuda", device)
        cfg = GupuvikConfig(spec.vocab, spec.width, len(spec.layers), spec.norm_eps, spec.embed_scale, VMX_F32 if dtype == "float32" else VMX_BF16,
                            block_size, num_blocks, max_tokens, max_seqs, self.state_slots)
        layers = (GupuvikLayerConfig * len(spec.layers))()
        for i, l in enumerate(spec.layers):
            layers[i] = GupuvikLayerConfig(MIXERS[l.mixer], l.heads, l.kv_heads, l.dim, l.vdim, l.window, l.keep_first, l.scale, l.softcap,
                                           -1 if l.kv_from is None else l.kv_from, l.conv, l.decay_rank, l.gate_rank, MLPS[l.mlp], l.ff, l.experts,
                                           l.top, l.expert_ff)
        self._h = C.c_void_p()
        check(lib.vmx_gupuvik_create(C.byref(cfg), layers, C.byref(self._h)))

    @classmethod
    def from_pretrained(cls, model_dir, dtype: str = "bfloat16", **kw) -> "GupuvikForCausalLM":
        from .checkpoint import CheckpointDir
        cfg = json.loads((Path(model_dir) / "config.json").read_text())
        ck = CheckpointDir(model_dir)
        try:
            shapes = {}
            for name, fn in ck.where.items():
                f = ck._file(fn)
                shapes[name] = f.info(lib.vmx_safetensors_find(f._h, name.encode()))[2]
        finally:
            ck.close()
        model = cls(GupuvikSpec.from_config(cfg, shapes), dtype=dtype, **kw)
        model.load_checkpoint(model_dir)
        return model

    def close(self):
        if self._h:
            lib.vmx_gupuvik_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _stream():
        return torch.cuda.current_stream().cuda_stream

    def load_tensor(self, name: str, t) -> None:
        """t: bf16 torch tensor (host or device) or a numpy uint16 array of bf16 bit patterns."""
        if isinstance(t, np.ndarray):
            assert t.dtype == np.uint16, f"{name}: bf16 bit patterns expected"
            t = np.ascontiguousarray(t)
            check(lib.vmx_gupuvik_load_tensor(self._h, name.encode(), t.ctypes.data, t.nbytes, self._stream()))
            return
        assert t.dtype == torch.bfloat16, f"{name}: bf16 expected, got {t.dtype}"
        t = t.contiguous()
        check(lib.vmx_gupuvik_load_tensor(self._h, name.encode(), t.data_ptr(), t.numel() * 2, self._stream()))

    def load_state(self, tensors: dict) -> None:
        for name, t in tensors.items():
            self.load_tensor(name, t)
        self.check_loaded()

    def check_loaded(self) -> None:
        if lib.vmx_gupuvik_missing_tensors(self._h) != 0:
            raise ValueError(lib.vmx_last_error().decode("utf-8", "replace"))

    def load_checkpoint(self, model_dir) -> None:
        """Every tensor of the directory's *.safetensors files under its own name (the library's safetensors reader)."""
        from .checkpoint import CheckpointDir
        ck = CheckpointDir(model_dir)
        try:
            for name in ck.where:
                f = ck._file(ck.where[name])
                dtype = f.info(lib.vmx_safetensors_find(f._h, name.encode()))[1]
                if dtype != "BF16":
                    raise ValueError(f"{model_dir}: tensor `{name}` is {dtype}; Gupuvik checkpoints hold bf16")
                m = re.fullmatch(r"l(\d+)\.rg2(\.b)?", name)
                if m and int(m.group(1)) < len(self.spec.layers) and self.spec.layers[int(m.group(1))].mlp is None:
                    continue                 # the gate of a feed-forward this layer does not have
                self.load_tensor(name, ck.get(name))
        finally:
            ck.close()
        self.check_loaded()

    def forward(self, tokens, prev_tokens, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits: bool = True,
                want_greedy: bool = False, layer_trace: bool = False, seq_starts=None, state_slots=None):
        """One packed step; every argument an int32 CUDA tensor ([T] each, block_tables [S, max_blocks], seq_starts [S + 1],
        state_slots [S], logit_rows [n]); prev_tokens is not used by this design.
        Returns (logits f32 [n, vocab] or None, greedy ids int32 [n] or None, trace f32 [layers, T, width] or None)."""
        if seq_starts is None or state_slots is None:
            raise ValueError("Gupuvik carries recurrent state: the step needs seq_starts and state_slots")
        T = tokens.numel()
        S = seq_starts.numel() - 1           # the sequences of THIS step; the block table may hold more rows
        if S < 1 or state_slots.numel() != S or block_tables.shape[0] < S:
            raise ValueError(f"Gupuvik: {S} sequences by seq_starts, {state_slots.numel()} state slots, {block_tables.shape[0]} block-table rows")
        if not all(a.numel() == T for a in (positions, slots, seq_ids)):
            raise ValueError("Gupuvik: tokens, positions, slots and seq_ids must have one entry per token")
        n = 0 if logit_rows is None else logit_rows.numel()
        logits = torch.empty((n, self.spec.vocab), dtype=torch.float32, device=self.device) if n else None
        ids = torch.empty(n, dtype=torch.int32, device=self.device) if (n and want_greedy) else None
        trace = torch.empty((len(self.spec.layers), T, self.spec.width), dtype=torch.float32, device=self.device) if layer_trace else None
        check(lib.vmx_gupuvik_forward(self._h, tokens.data_ptr(), positions.data_ptr(), slots.data_ptr(), seq_ids.data_ptr(), T,
                                      block_tables.data_ptr(), S, block_tables.shape[1], seq_starts.data_ptr(),
                                      state_slots.data_ptr(), None if not n else logit_rows.data_ptr(), n,
                                      None if logits is None else logits.data_ptr(), None if ids is None else ids.data_ptr(),
                                      None if trace is None else trace.data_ptr(), self._stream()))
        return (logits if want_logits else None), ids, trace
