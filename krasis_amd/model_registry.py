"""Model registry: config.json -> the class that serves the checkpoint.

Two families of engines live in this package:
  * `CpuDecoder` (decode_setup.py): the quantized single-request decode graph of the HF model types (`model_type` in config.json);
  * `BatchEngine` (scheduler.py): the batched serving store for designs described layer by layer (`architecture` in config.json), bf16 / f32
    weights, paged cache, several requests per step.
`load_model(model_dir, ...)` picks by config.json.  A new layer-described design registers a function that turns its config.json into
`LayerSpec`s and names its tensors (`register_architecture`); the mechanisms themselves (rotation, unit norm, window, sink, borrowed cache,
group-limited router, clamped gated activation) are parameters of the serving store, not code of the design."""
from __future__ import annotations

import json
import os
import struct
from dataclasses import dataclass
from typing import Callable, Dict, Iterator, List, Optional, Tuple

import numpy as np

from . import serve_store as S


# ------------------------------------------------------------------------------------------------------------------------------------
# safetensors without a tensor library: 8-byte little-endian header length, JSON header (name -> dtype, shape, data_offsets), raw data
# ------------------------------------------------------------------------------------------------------------------------------------
class SafetensorsFile:
    _DT = {"BF16": (np.uint16, 2), "F32": (np.float32, 4), "I32": (np.int32, 4), "F16": (np.float16, 2), "I64": (np.int64, 8)}

    def __init__(self, path: str):
        self.path = path
        with open(path, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            if n > (1 << 30):
                raise IOError(f"{path}: header of {n} bytes")
            self.meta = json.loads(f.read(n))
        self.meta.pop("__metadata__", None)
        self._base = 8 + n
        self._map = np.memmap(path, dtype=np.uint8, mode="r")

    def names(self) -> List[str]:
        return list(self.meta)

    def has(self, name: str) -> bool:
        return name in self.meta

    def shape(self, name: str) -> Tuple[int, ...]:
        return tuple(self.meta[name]["shape"])

    def get(self, name: str) -> np.ndarray:
        """BF16 tensors come back as uint16 bit patterns, F32 as float32 (what ServeStore.set_tensor takes)"""
        m = self.meta.get(name)
        if m is None:
            raise IOError(f"tensor {name} not found in {self.path}")
        if m["dtype"] not in self._DT:
            raise IOError(f"tensor {name}: dtype {m['dtype']} not handled")
        dt, sz = self._DT[m["dtype"]]
        lo, hi = m["data_offsets"]
        n = int(np.prod(m["shape"])) if m["shape"] else 1
        if hi - lo != n * sz:
            raise IOError(f"tensor {name}: {hi - lo} bytes for shape {m['shape']}")
        a = np.frombuffer(self._map, dtype=dt, count=n, offset=self._base + lo).reshape(m["shape"])
        if m["dtype"] == "F16":
            a = a.astype(np.float32)
        return a


# ------------------------------------------------------------------------------------------------------------------------------------
# layer-described designs
# ------------------------------------------------------------------------------------------------------------------------------------
@dataclass
class ServeModelSpec:
    vocab: int
    width: int
    norm_kind: int
    norm_eps: float
    layers: List[S.LayerSpec]
    tensors: Callable[["ServeModelSpec"], Iterator[Tuple[int, str, int, str]]]      # (layer, role, index, tensor name)


_ARCHITECTURES: Dict[str, Callable[[dict], ServeModelSpec]] = {}


def register_architecture(name: str, spec_from_config: Callable[[dict], ServeModelSpec]) -> None:
    _ARCHITECTURES[name] = spec_from_config


def architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


# ---- Lomutar: pre-norm layers with ONE layer norm (weight + bias) feeding an attention mixer and a feed-forward in parallel.  Attention: grouped
# key / value heads, interleaved partial rotary with linear position scaling, weightless RMS norm of q and k after the rotation, sliding window,
# a learned per-head sink in the softmax denominator, optional reuse of an earlier layer's cache.  Feed-forward: gated tanh-GELU, or a mixture of
# clamped gated experts behind a softmax router restricted to the best groups, plus a shared expert.
def _lomutar_tensors(spec: ServeModelSpec) -> Iterator[Tuple[int, str, int, str]]:
    yield -1, "embed", 0, "embed"
    yield -1, "final_norm_w", 0, "final.norm"
    yield -1, "final_norm_b", 0, "final.norm.b"
    yield -1, "head", 0, "head"
    for i, l in enumerate(spec.layers):
        p = f"l{i}"
        yield i, "norm_w", 0, f"{p}.norm1"
        yield i, "norm_b", 0, f"{p}.norm1.b"
        yield i, "q", 0, f"{p}.mix.q"
        if l.kv_from < 0:
            yield i, "k", 0, f"{p}.mix.k"
            yield i, "v", 0, f"{p}.mix.v"
        yield i, "o", 0, f"{p}.mix.o"
        if l.has_sink:
            yield i, "sink", 0, f"{p}.mix.sink"
        if l.mlp_kind == S.MLP_DENSE:
            for r in ("gate", "up", "down"):
                yield i, r, 0, f"{p}.mlp.{r}"
        elif l.mlp_kind == S.MLP_MOE:
            yield i, "router", 0, f"{p}.mlp.router"
            for e in range(l.experts):
                for r in ("gate", "up", "down"):
                    yield i, f"expert_{r}", e, f"{p}.mlp.e{e}.{r}"
            if l.shared_ff:
                for r in ("gate", "up", "down"):
                    yield i, f"shared_{r}", 0, f"{p}.mlp.shared.{r}"


def lomutar_spec(cfg: dict) -> ServeModelSpec:
    layers: List[S.LayerSpec] = []
    for i, lc in enumerate(cfg["layers"]):
        if lc.get("type", "attention") != "attention":
            raise ValueError(f"layer {i}: mixer type {lc.get('type')!r} is not part of this design")
        m = lc["mixer"]
        rot = m.get("rot") or {}
        sc = (rot.get("scaling") or {})
        l = S.LayerSpec(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                        rot_dims=int(rot.get("dims", 0)), rot_interleaved=1, rot_base=float(rot.get("base", 10000.0)), rot_factor=float(sc.get("factor", 1.0)),
                        qk_unit_norm=1, scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size", 0)), has_sink=1,
                        kv_from=-1 if m.get("kv_from") is None else int(m["kv_from"]))
        mlp = lc.get("mlp")
        if mlp is not None:
            kind = mlp.get("kind")
            if kind == "dense":
                l.mlp_kind, l.ff, l.dense_act = S.MLP_DENSE, int(mlp["ff"]), S.ACT_GELU_TANH
            elif kind == "moe":
                r, ex = mlp["router"], mlp["expert"]
                g = r.get("groups") or {}
                l.mlp_kind, l.experts, l.top = S.MLP_MOE, int(r["experts"]), int(r["top"])
                l.groups, l.keep, l.renorm = int(g.get("count", 1)), int(g.get("keep", g.get("count", 1))), 0
                l.expert_ff, l.expert_act, l.expert_limit, l.expert_alpha = int(ex["ff"]), S.ACT_CLAMPED_SWIGLU, float(ex["limit"]), 1.702
                sh = mlp.get("shared")
                if sh:
                    l.shared_ff, l.shared_limit = int(sh["ff"]), float(sh["limit"])
            else:
                raise ValueError(f"layer {i}: feed-forward kind {kind!r}")
        layers.append(l)
    return ServeModelSpec(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_kind=S.NORM_LAYER, norm_eps=float(cfg["norm"]["eps"]), layers=layers,
                          tensors=_lomutar_tensors)


register_architecture("Lomutar", lomutar_spec)


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def model_family(cfg: dict) -> str:
    """'serve:<architecture>' for a layer-described design, 'decode:<model_type>' for the HF model types of the quantized decode graph"""
    arch = cfg.get("architecture")
    if isinstance(arch, str) and arch in _ARCHITECTURES:
        return "serve:" + arch
    if "model_type" in cfg or "text_config" in cfg or "language_config" in cfg:
        return "decode:" + str(cfg.get("model_type", ""))
    raise ValueError(f"config.json names no known design (architecture {arch!r}; known: {architectures()})")


def load_model(model_dir: str, dtype: str = "bfloat16", max_tokens: int = 4096, max_slots: int = 4, device: int = 0, build: bool = False, **decoder_args):
    """The serving object for a checkpoint directory: a `BatchEngine` (layer-described designs) or a `CpuDecoder` with its weights initialised."""
    cfg = read_config(model_dir)
    fam = model_family(cfg)
    if fam.startswith("serve:"):
        from .scheduler import BatchEngine
        spec = _ARCHITECTURES[fam[6:]](cfg)
        eng = BatchEngine(spec, dtype=dtype, max_tokens=max_tokens, max_slots=max_slots, device=device, build=build)
        eng.load_safetensors(os.path.join(model_dir, "model.safetensors"))
        return eng
    from .decode_setup import CpuDecoder
    dec = CpuDecoder(model_dir, device=device, **decoder_args)
    dec.init_weights(max_rope_seq=max(max_tokens, 8192))
    return dec
