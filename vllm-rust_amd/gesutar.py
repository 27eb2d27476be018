"""Host-side driver of the Gesutar decoder family (libvmx `vmx_gesutar_*`).

A Gesutar model is a stack of pre-norm layers listed in its config.json, each a token mixer ("latent_attention": low-rank
compressed keys/values, sliding window, per-head softmax sink, sigmoid output gate) and an optional feed-forward ("moe": softmax
router with group-limited top-k, squared-ReLU experts, shared expert); a hashed bigram table is added to the token embedding.
This file reads the configuration, hands the checkpoint's tensors to the library under their file names and wraps the one
forward entry point, which takes a step's tokens packed (prompts of unequal length, prompt portions and decode tokens alike).
All arithmetic happens in the library.
"""
from __future__ import annotations

import ctypes as C
import dataclasses
import json
import math
from pathlib import Path

import numpy as np
import torch

from ._lib import GesutarConfig, GesutarLayerConfig, check, lib

VMX_F32, VMX_BF16 = 0, 1
MIXERS = {"latent_attention": 0}
MLPS = {None: 0, "moe": 1}


@dataclasses.dataclass
class GesutarLayerSpec:
    mixer: str = "latent_attention"
    heads: int = 4
    dim: int = 32
    rot_dim: int = 16
    vdim: int = 32
    kv_rank: int = 64
    window: int = 64
    rot_dims: int = 16
    rot_base: float = 10000.0
    scale: float = 0.125
    mlp: str | None = "moe"
    experts: int = 8
    top: int = 2
    groups: int = 1
    keep_groups: int = 1
    expert_ff: int = 64
    shared_ff: int = 0
    router_scale: float = 1.0

    @staticmethod
    def from_config(entry: dict) -> "GesutarLayerSpec":
        kind = entry["type"]
        if kind not in MIXERS:
            raise ValueError(f"Gesutar: unknown layer type `{kind}`")
        m = entry["mixer"]
        rot = m.get("rot") or {}
        s = GesutarLayerSpec(mixer=kind, heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                             kv_rank=int(m["kv_rank"]), window=int(m["mask"]["size"]), rot_dims=int(rot.get("dims", m["rot_dim"])),
                             rot_base=float(rot.get("base", 10000.0)), scale=float(m["scale"]), mlp=None)
        ff = entry.get("mlp")
        if ff is not None:
            if ff.get("kind", "moe") != "moe":
                raise ValueError(f"Gesutar: unknown feed-forward kind `{ff.get('kind')}`")
            r = ff["router"]
            g = r.get("groups") or {}
            shared = ff.get("shared") or {}
            s.mlp, s.experts, s.top = "moe", int(r["experts"]), int(r["top"])
            s.groups, s.keep_groups = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1)))
            s.expert_ff, s.shared_ff, s.router_scale = int(ff["expert"]["ff"]), int(shared.get("ff", 0)), float(r.get("scale", 1.0))
        return s

    def to_config(self) -> dict:
        e = {"type": self.mixer,
             "mixer": {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "kv_rank": self.kv_rank,
                       "mask": {"size": self.window}, "rot": {"base": self.rot_base, "dims": self.rot_dims}, "scale": self.scale},
             "mlp": None}
        if self.mlp == "moe":
            e["mlp"] = {"kind": "moe", "expert": {"ff": self.expert_ff},
                        "router": {"experts": self.experts, "top": self.top, "scale": self.router_scale,
                                   "groups": {"count": self.groups, "keep": self.keep_groups}}}
            if self.shared_ff:
                e["mlp"]["shared"] = {"ff": self.shared_ff}
        return e


@dataclasses.dataclass
class GesutarSpec:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-5
    embed_scale: float = 1.0
    bigram_buckets: int = 0
    bigram_mul_prev: int = 0
    bigram_mul_cur: int = 0

    @staticmethod
    def from_config(cfg: dict) -> "GesutarSpec":
        emb = cfg.get("embedding") or {}
        bg = emb.get("bigram") or {}
        return GesutarSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), layers=[GesutarLayerSpec.from_config(e) for e in cfg["layers"]],
                           norm_eps=float(cfg["norm"]["eps"]), embed_scale=float(emb.get("scale", 1.0)), bigram_buckets=int(bg.get("buckets", 0)),
                           bigram_mul_prev=int(bg.get("mul_prev", 0)), bigram_mul_cur=int(bg.get("mul_cur", 0)))

    def to_config(self) -> dict:
        return {"architecture": "Gesutar", "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "embedding": {"scale": self.embed_scale, "bigram": {"buckets": self.bigram_buckets, "mul_prev": self.bigram_mul_prev,
                                                                     "mul_cur": self.bigram_mul_cur}},
                "layers": [l.to_config() for l in self.layers]}

    def tensor_shapes(self) -> dict:
        """Name -> shape of every checkpoint tensor, in file order."""
        W, out = self.width, {}
        out["embed"] = (self.vocab, W)
        if self.bigram_buckets:
            out["bigram"] = (self.bigram_buckets + 1, W)
        for i, l in enumerate(self.layers):
            p = f"l{i}."
            out[p + "norm1"] = (W,)
            if l.mlp:
                out[p + "norm2"] = (W,)
            out[p + "mix.q"] = (l.heads * (l.dim + l.rot_dim), W)
            out[p + "mix.dkv"] = (l.kv_rank + l.rot_dim, W)
            out[p + "mix.dkv.norm"] = (l.kv_rank,)
            out[p + "mix.uk"] = (l.heads * l.dim, l.kv_rank)
            out[p + "mix.uv"] = (l.heads * l.vdim, l.kv_rank)
            out[p + "mix.sink"] = (l.heads,)
            out[p + "mix.g"] = (l.heads * l.vdim, W)
            out[p + "mix.o"] = (W, l.heads * l.vdim)
            if l.mlp:
                for e in range(l.experts):
                    out[p + f"mlp.e{e}.up"] = (l.expert_ff, W)
                    out[p + f"mlp.e{e}.down"] = (W, l.expert_ff)
                out[p + "mlp.router"] = (l.experts, W)
                if l.shared_ff:
                    out[p + "mlp.shared.up"] = (l.shared_ff, W)
                    out[p + "mlp.shared.down"] = (W, l.shared_ff)
        out["final.norm"] = (W,)
        out["head"] = (self.vocab, W)
        return out


def synthetic_weights(spec: GesutarSpec, seed: int = 0, device="cpu") -> dict:
    """Seeded random-init checkpoint of the architecture (bf16 tensors on `device`): matrices ~ 1 / sqrt(in), norm weights
    around 1, sinks around 0, so that activations stay O(1) through the stack."""
    g = torch.Generator(device=device).manual_seed(seed)

    def randn(shape):
        return torch.randn(shape, generator=g, device=device)
    ck = {}
    for name, shape in spec.tensor_shapes().items():
        if name.endswith("norm1") or name.endswith("norm2") or name.endswith(".norm"):
            t = 1.0 + 0.1 * randn(shape)
        elif name.endswith("sink"):
            t = 0.5 * randn(shape)
        elif name in ("embed", "bigram"):
            t = randn(shape) * (0.5 if name == "bigram" else 1.0 / max(spec.embed_scale, 1e-6))
        else:
            t = randn(shape) / math.sqrt(shape[-1])
        ck[name] = t.to(torch.bfloat16)
    return ck


class GesutarForCausalLM:
    """The executor handle: weights, paged latent cache and workspaces live in the library."""

    architecture = "Gesutar"

    def __init__(self, spec: GesutarSpec, dtype: str = "bfloat16", block_size: int = 16, num_blocks: int = 256, max_tokens: int = 2048,
                 max_seqs: int = 64, device: int = 0):
        if dtype not in ("bfloat16", "float32"):
            raise ValueError(f"Gesutar runs in bfloat16 or float32, not `{dtype}`")
        self.spec, self.dtype = spec, dtype
        self.block_size, self.num_blocks, self.max_tokens, self.max_seqs = block_size, num_blocks, max_tokens, max_seqs
        self.vocab_size = spec.vocab
        self.device = torch.device("cuda", device)
        cfg = GesutarConfig(spec.vocab, spec.width, len(spec.layers), spec.norm_eps, spec.embed_scale, spec.bigram_buckets, spec.bigram_mul_prev,
                            spec.bigram_mul_cur, VMX_F32 if dtype == "float32" else VMX_BF16, block_size, num_blocks, max_tokens, max_seqs)
        layers = (GesutarLayerConfig * len(spec.layers))()
        for i, l in enumerate(spec.layers):
            layers[i] = GesutarLayerConfig(MIXERS[l.mixer], l.heads, l.dim, l.rot_dim, l.vdim, l.kv_rank, l.window, l.rot_dims, l.rot_base, l.scale,
                                           MLPS[l.mlp], l.experts, l.top, l.groups, l.keep_groups, l.expert_ff, l.shared_ff, l.router_scale)
        self._h = C.c_void_p()
        check(lib.vmx_gesutar_create(C.byref(cfg), layers, C.byref(self._h)))

    @classmethod
    def from_pretrained(cls, model_dir, dtype: str = "bfloat16", **kw) -> "GesutarForCausalLM":
        cfg = json.loads((Path(model_dir) / "config.json").read_text())
        model = cls(GesutarSpec.from_config(cfg), dtype=dtype, **kw)
        model.load_checkpoint(model_dir)
        return model

    def close(self):
        if self._h:
            lib.vmx_gesutar_destroy(self._h)
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
            check(lib.vmx_gesutar_load_tensor(self._h, name.encode(), t.ctypes.data, t.nbytes, self._stream()))
            return
        assert t.dtype == torch.bfloat16, f"{name}: bf16 expected, got {t.dtype}"
        t = t.contiguous()
        check(lib.vmx_gesutar_load_tensor(self._h, name.encode(), t.data_ptr(), t.numel() * 2, self._stream()))

    def load_state(self, tensors: dict) -> None:
        for name, t in tensors.items():
            self.load_tensor(name, t)
        self.check_loaded()

    def check_loaded(self) -> None:
        if lib.vmx_gesutar_missing_tensors(self._h) != 0:
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
                    raise ValueError(f"{model_dir}: tensor `{name}` is {dtype}; Gesutar checkpoints hold bf16")
                self.load_tensor(name, ck.get(name))
        finally:
            ck.close()
        self.check_loaded()

    def forward(self, tokens, prev_tokens, positions, slots, seq_ids, block_tables, logit_rows=None, want_logits: bool = True,
                want_greedy: bool = False, layer_trace: bool = False):
        """One packed step; every argument an int32 CUDA tensor ([T] each, block_tables [S, max_blocks], logit_rows [n]).
        Returns (logits f32 [n, vocab] or None, greedy ids int32 [n] or None, trace f32 [layers, T, width] or None)."""
        T = tokens.numel()
        n = 0 if logit_rows is None else logit_rows.numel()
        logits = torch.empty((n, self.spec.vocab), dtype=torch.float32, device=self.device) if n else None
        ids = torch.empty(n, dtype=torch.int32, device=self.device) if (n and want_greedy) else None
        trace = torch.empty((len(self.spec.layers), T, self.spec.width), dtype=torch.float32, device=self.device) if layer_trace else None
        check(lib.vmx_gesutar_forward(self._h, tokens.data_ptr(), prev_tokens.data_ptr(), positions.data_ptr(), slots.data_ptr(),
                                      seq_ids.data_ptr(), T, block_tables.data_ptr(), block_tables.shape[0], block_tables.shape[1],
                                      None if not n else logit_rows.data_ptr(), n, None if logits is None else logits.data_ptr(),
                                      None if ids is None else ids.data_ptr(), None if trace is None else trace.data_ptr(), self._stream()))
        return (logits if want_logits else None), ids, trace
