"""Gitopel: a decoder stack that interleaves two token mixers, chosen per layer by the checkpoint's config.json:

* ``attention`` -- sliding-window attention with mean-pooled blocks behind the window, sigmoid weights, grouped query
  heads whose values are the key projection, interleaved partial rotary, unit-RMS q / k, a per-head score bias and a
  per-head sigmoid output gate;
* ``gla`` -- gated linear attention with a low-rank, temperature-flattened decay per key channel, an RMS norm per head on
  the read-out and a SiLU gate;

every sublayer wrapped as ``x + norm_after(f(norm_before(x)))`` with grouped RMS norms, gated SiLU feed-forwards on the
layers that have one, a final grouped norm and an untied head.

This file only TRANSLATES the design -- config.json keys, tensor names, how the per-sublayer matrices are fused -- into
the generic sequence-mixer runtime (models/seqmix.py); every mechanism lives there and in csrc/seq_*.hip with its
constants as parameters.
"""
from __future__ import annotations

import json
import os

import torch

from .config import GLACfg, PooledWindowAttnCfg, SeqLayerCfg, SeqMixCfg
from .seqmix import SeqMixLM

ARCHITECTURE = "Gitopel"


def config_from_dict(c: dict, name: str = "gitopel") -> SeqMixCfg:
    layers = []
    for entry in c["layers"]:
        m, kind = entry["mixer"], entry["type"]
        if kind == "attention":
            mixer = PooledWindowAttnCfg(heads=m["heads"], kv_heads=m["kv_heads"], dim=m["dim"], vdim=m["vdim"],
                                        window=m["mask"]["size"], pool=m["mask"]["pool"], rot_dims=m["rot"]["dims"],
                                        rot_base=float(m["rot"]["base"]), scale=float(m["scale"]))
        elif kind == "gla":
            mixer = GLACfg(heads=m["heads"], dim=m["dim"], vdim=m["vdim"], tau=float(m["tau"]))
        else:
            raise ValueError(f"{ARCHITECTURE}: unknown mixer type '{kind}'")
        mlp = entry.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"{ARCHITECTURE}: unknown feed-forward kind '{mlp.get('kind')}'")
        layers.append(SeqLayerCfg(mixer=mixer, ff=int(mlp["ff"]) if mlp is not None else 0))
    return SeqMixCfg(vocab_size=c["vocab"], width=c["width"], norm_eps=float(c["norm"]["eps"]),
                     norm_groups=int(c["norm"]["groups"]), layers=layers, name=name, architecture=ARCHITECTURE)


def config_from_dir(path: str) -> SeqMixCfg:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))


def tensor_shapes(cfg: SeqMixCfg, rank: int = 16) -> dict:
    """checkpoint tensor name -> shape (linear weights are [out, in])"""
    W, sh = cfg.width, {"embed": (cfg.vocab_size, cfg.width), "final.norm": (cfg.width,), "head": (cfg.vocab_size, cfg.width)}
    for i, ly in enumerate(cfg.layers):
        p, m = f"l{i}.", ly.mixer
        sh[p + "norm1"], sh[p + "norm1b"] = (W,), (W,)
        if m.kind == "attention":
            sh.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.q.b": (m.heads * m.dim,),
                       p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.k.b": (m.kv_heads * m.dim,),
                       p + "mix.pb": (m.heads,), p + "mix.g": (m.heads, W),
                       p + "mix.o": (W, m.heads * m.vdim), p + "mix.o.b": (W,)})
        else:
            r = m.rank or rank
            sh.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W),
                       p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                       p + "mix.o": (W, m.heads * m.vdim), p + "mix.norm": (m.vdim,),
                       p + "mix.a1": (r, W), p + "mix.a2": (m.heads * m.dim, r), p + "mix.a2.b": (m.heads * m.dim,)})
        if ly.ff:
            sh.update({p + "norm2": (W,), p + "norm2b": (W,), p + "mlp.gate": (ly.ff, W), p + "mlp.up": (ly.ff, W),
                       p + "mlp.down": (W, ly.ff)})
    return sh


def synth_state(cfg: SeqMixCfg, seed: int = 0, rank: int = 16) -> dict:
    """Seeded random fp32 checkpoint of the design (tests, benchmarks): name -> tensor."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        leaf = name.split(".", 1)[-1] if name[0] == "l" and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "norm1b", "norm2b", "final.norm", "mix.norm"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf.endswith(".b") or leaf == "mix.pb":
            t = 0.5 * torch.randn(shape, generator=g)
        elif leaf == "mix.a2":
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        else:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        sd[name] = t
    return sd


class Gitopel(SeqMixLM):
    """``AutoModelLM`` resolves a directory whose config.json says ``"architecture": "Gitopel"`` to this class."""

    @staticmethod
    def read_config(path: str) -> SeqMixCfg:
        return config_from_dir(path)

    def layer_tensors(self, i: int, ly: SeqLayerCfg, get):
        """The design's tensor names -> the runtime's fused per-layer tensors.  ``get(name)`` fetches one checkpoint
        tensor in the storage dtype on the device."""
        p, m = f"l{i}.", ly.mixer
        t = {"norm1": get(p + "norm1"), "norm1b": get(p + "norm1b")}
        if m.kind == "attention":
            q, k, g = get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.g")
            t["proj_w"] = torch.cat([q, k, g], dim=0)                       # [q | k | gate]
            t["proj_b"] = torch.cat([get(p + "mix.q.b"), get(p + "mix.k.b"), torch.zeros_like(g[:, 0])])
            t["pos_bias"] = get(p + "mix.pb")
            t["out_w"], t["out_b"] = get(p + "mix.o"), get(p + "mix.o.b")
        else:
            a1 = get(p + "mix.a1")
            m.rank = a1.shape[0]
            t["proj_w"] = torch.cat([get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"), get(p + "mix.g"), a1], dim=0)
            t["proj_b"] = None
            t["a2_w"], t["a2_b"] = get(p + "mix.a2"), get(p + "mix.a2.b")
            t["head_norm"] = get(p + "mix.norm")
            t["out_w"], t["out_b"] = get(p + "mix.o"), None
        if ly.ff:
            t["norm2"], t["norm2b"] = get(p + "norm2"), get(p + "norm2b")
            t["gu_w"] = torch.cat([get(p + "mlp.gate"), get(p + "mlp.up")], dim=0)
            t["down_w"] = get(p + "mlp.down")
        return t

    def top_tensors(self, get):
        return {"embed": get("embed"), "final_norm": get("final.norm"), "head": get("head")}
