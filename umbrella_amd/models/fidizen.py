"""Fidizen: a decoder stack of latent-attention layers with dense or routed feed-forwards, chosen per layer by the
checkpoint's config.json:

* every sublayer reads the residual stream itself, through a short causal convolution over time (``h + conv(h)``, one
  filter per channel), and only its OUTPUT is normed: ``x + norm(f(h))``; the embedding is scaled by a constant;
* ``latent_attention`` -- softmax attention whose queries go through a normed low-rank latent and whose keys and values
  come from one normed low-rank latent per token plus one rotated key part shared by the heads (only those are cached);
  interleaved rotary on the rotated parts, a sliding window, a learned sink per head in the softmax denominator and a
  sigmoid output gate computed from the mixer's input;
* feed-forwards: dense with the PolyNorm activation, or routed experts (sigmoid scores, top-k, the score multiplies the
  chosen expert's input) beside an always-on shared expert, all gated SiLU;
* a layer may name another layer whose tensors it uses (``weights_of``) while keeping a cache and state of its own.

This file only TRANSLATES the design -- config.json keys, tensor names, how matrices are fused or stacked -- into the
generic sequence-mixer runtime (models/seqmix.py); every mechanism lives there and in csrc/seq_*.hip with its constants as
parameters.
"""
from __future__ import annotations

import json
import os

import torch

from .config import LatentAttnCfg, SeqLayerCfg, SeqMixCfg
from .seqmix import SeqMixLM

ARCHITECTURE = "Fidizen"


def _layer(entry: dict) -> SeqLayerCfg:
    m, kind = entry["mixer"], entry["type"]
    if kind != "latent_attention":
        raise ValueError(f"{ARCHITECTURE}: unknown mixer type '{kind}'")
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    rot_dim = int(m.get("rot_dim", 0))
    mixer = LatentAttnCfg(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=rot_dim, vdim=int(m["vdim"]),
                          q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), window=int(mask.get("size", 0)),
                          rot_dims=int(rot.get("dims", rot_dim)), rot_base=float(rot.get("base", 10000.0)),
                          scale=float(m["scale"]))
    if mixer.rot_dims > mixer.rot_dim or mixer.rot_dims % 2:
        raise ValueError(f"{ARCHITECTURE}: rot.dims must be even and at most rot_dim")
    mlp = entry.get("mlp")
    wo = entry.get("weights_of")
    wo = int(wo) if wo is not None else None
    if mlp is None:
        return SeqLayerCfg(mixer=mixer, ff=0, weights_of=wo)
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return SeqLayerCfg(mixer=mixer, ff=int(mlp["ff"]), ff_kind="polynorm", weights_of=wo)
    if kind == "moe":
        shared = mlp.get("shared")
        return SeqLayerCfg(mixer=mixer, ff=0, ff_kind="moe", experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                           expert_ff=int(mlp["expert"]["ff"]), shared_ff=int(shared["ff"]) if shared else 0, weights_of=wo)
    raise ValueError(f"{ARCHITECTURE}: unknown feed-forward kind '{kind}'")


def config_from_dict(c: dict, name: str = "fidizen") -> SeqMixCfg:
    return SeqMixCfg(vocab_size=int(c["vocab"]), width=int(c["width"]), norm_eps=float(c["norm"]["eps"]), norm_groups=1,
                     layers=[_layer(e) for e in c["layers"]], name=name, architecture=ARCHITECTURE,
                     embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)), pre_norm=False,
                     canon_taps=int((c.get("canon") or {}).get("taps", 1)))


def config_from_dir(path: str) -> SeqMixCfg:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))


def tensor_shapes(cfg: SeqMixCfg) -> dict:
    """checkpoint tensor name -> shape (linear weights are [out, in]); layers that use another layer's tensors have none"""
    W, sh = cfg.width, {"embed": (cfg.vocab_size, cfg.width), "final.norm": (cfg.width,), "head": (cfg.vocab_size, cfg.width)}
    for i, ly in enumerate(cfg.layers):
        if ly.weights_of is not None:
            continue
        p, m = f"l{i}.", ly.mixer
        sh.update({p + "norm1": (W,), p + "canon1": (W, cfg.canon_taps),
                   p + "mix.dq": (m.q_rank, W), p + "mix.dq.norm": (m.q_rank,), p + "mix.uq": (m.heads * (m.dim + m.rot_dim), m.q_rank),
                   p + "mix.dkv": (m.kv_rank + m.rot_dim, W), p + "mix.dkv.norm": (m.kv_rank,),
                   p + "mix.uk": (m.heads * m.dim, m.kv_rank), p + "mix.uv": (m.heads * m.vdim, m.kv_rank),
                   p + "mix.sink": (m.heads,), p + "mix.g": (m.heads * m.vdim, W), p + "mix.o": (W, m.heads * m.vdim)})
        if not ly.has_ff:
            continue
        sh.update({p + "norm2": (W,), p + "canon2": (W, cfg.canon_taps)})
        if ly.ff_kind == "polynorm":
            sh.update({p + "mlp.up": (ly.ff, W), p + "mlp.down": (W, ly.ff), p + "mlp.act": (4,)})
        else:
            sh[p + "mlp.router"] = (ly.experts, W)
            for e in [f"e{k}" for k in range(ly.experts)] + (["shared"] if ly.shared_ff else []):
                f = ly.shared_ff if e == "shared" else ly.expert_ff
                sh.update({p + f"mlp.{e}.gate": (f, W), p + f"mlp.{e}.up": (f, W), p + f"mlp.{e}.down": (W, f)})
    return sh


def synth_state(cfg: SeqMixCfg, seed: int = 0) -> dict:
    """Seeded random fp32 checkpoint of the design (tests, benchmarks): name -> tensor."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[-1] if name[0] == "l" and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "final.norm", "mix.dq.norm", "mix.dkv.norm"):
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "embed":
            t = torch.randn(shape, generator=g)
        elif leaf == "mix.sink":
            t = torch.randn(shape, generator=g)
        elif leaf == "mlp.act":
            t = torch.tensor([0.6, 0.3, 0.1, 0.05]) + 0.05 * torch.randn(shape, generator=g)
        elif leaf in ("canon1", "canon2"):
            t = 0.3 * torch.randn(shape, generator=g)
        elif leaf == "mlp.router":
            t = 2.0 * torch.randn(shape, generator=g) / shape[1] ** 0.5
        else:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
        sd[name] = t
    return sd


class Fidizen(SeqMixLM):
    """``AutoModelLM`` resolves a directory whose config.json says ``"architecture": "Fidizen"`` to this class."""

    @staticmethod
    def read_config(path: str) -> SeqMixCfg:
        return config_from_dir(path)

    def layer_tensors(self, i: int, ly: SeqLayerCfg, get):
        """The design's tensor names -> the runtime's fused per-layer tensors.  ``get(name)`` fetches one checkpoint
        tensor in the storage dtype on the device."""
        p, m = f"l{i}.", ly.mixer
        H, D, R = m.heads, m.dim, m.rot_dim
        t = {"norm1": None, "norm1b": get(p + "norm1"), "canon1": get(p + "canon1")}
        t["proj_w"] = torch.cat([get(p + "mix.dq"), get(p + "mix.dkv"), get(p + "mix.g")], dim=0)      # [dq | dkv | gate]
        t["dq_norm"], t["dkv_norm"], t["sink"] = get(p + "mix.dq.norm"), get(p + "mix.dkv.norm"), get(p + "mix.sink")
        t["uq_w"] = get(p + "mix.uq")
        # W_uk [heads dim][kv_rank] -> per head transposed [kv_rank][dim]: the weight of "carry the query into latent space"
        t["uk_t"] = get(p + "mix.uk").view(H, D, m.kv_rank).transpose(1, 2).contiguous()
        t["uv_w"] = get(p + "mix.uv")
        t["out_w"] = get(p + "mix.o")
        assert tuple(t["uq_w"].shape) == (H * (D + R), m.q_rank) and tuple(t["uv_w"].shape) == (H * m.vdim, m.kv_rank)
        if not ly.has_ff:
            return t
        t["norm2"], t["norm2b"], t["canon2"] = None, get(p + "norm2"), get(p + "canon2")
        if ly.ff_kind == "polynorm":
            t["gu_w"], t["down_w"], t["act"] = get(p + "mlp.up"), get(p + "mlp.down"), get(p + "mlp.act")
        else:
            t["router_w"] = get(p + "mlp.router")
            names = [f"mlp.e{k}" for k in range(ly.experts)]
            t["e_gu"] = torch.stack([torch.cat([get(p + n + ".gate"), get(p + n + ".up")], dim=0) for n in names])   # [E][2 F][W]
            t["e_down"] = torch.stack([get(p + n + ".down") for n in names])                                         # [E][W][F]
            if ly.shared_ff:
                t["s_gu_w"] = torch.cat([get(p + "mlp.shared.gate"), get(p + "mlp.shared.up")], dim=0)
                t["s_down_w"] = get(p + "mlp.shared.down")
        return t

    def top_tensors(self, get):
        return {"embed": get("embed"), "final_norm": get("final.norm"), "head": get("head")}
