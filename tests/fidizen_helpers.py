"""Tiny Fidizen configurations, seeded checkpoints and comparison helpers for the tests of that design."""
import torch

from umbrella_amd.models import fidizen


def layer(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=10, kv_rank=12, window=5, rot_dims=None, base=100.0, scale=None, mlp="dense",
          ff=24, experts=5, top=2, expert_ff=12, shared_ff=10, weights_of=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "rot": {"dims": rot_dim if rot_dims is None else rot_dims, "base": base},
         "scale": (dim + rot_dim) ** -0.5 if scale is None else scale}
    if window:
        m["mask"] = {"size": window}
    if mlp == "dense":
        f = {"kind": "dense", "ff": ff}
    elif mlp == "moe":
        f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff}}
        if shared_ff:
            f["shared"] = {"ff": shared_ff}
    else:
        f = None
    e = {"type": "latent_attention", "mixer": m, "mlp": f}
    if weights_of is not None:
        e["weights_of"] = weights_of
    return e


def config(layers, vocab=90, width=40, taps=3, eps=1e-5, embed_scale=3.0):
    return {"architecture": "Fidizen", "layers": layers, "norm": {"eps": eps}, "canon": {"taps": taps},
            "embedding": {"scale": embed_scale}, "vocab": vocab, "width": width}


# shapes that differ from one another in every size: layer order, sharing, odd sizes (nothing a multiple of 8), partial
# rotation, window 1 and no window, one expert used of many and all experts used, no shared expert, no feed-forward,
# latents wider than one lane pass, one tap (no history) and five
CONFIGS = {
    "mixed": config([layer(), layer(mlp="moe"), layer(weights_of=0), layer(mlp="moe", top=1, shared_ff=0, experts=7, heads=2, window=9),
                     layer(mlp=None, window=0, kv_rank=32, heads=8), layer(mlp="moe", weights_of=1)]),
    "odd": config([layer(heads=5, dim=6, rot_dim=6, rot_dims=4, vdim=10, q_rank=7, kv_rank=9, window=1, mlp="moe", experts=3, top=3,
                         expert_ff=5, shared_ff=7),
                   layer(heads=1, dim=3, rot_dim=2, vdim=5, q_rank=3, kv_rank=70, window=4, ff=17)],
                  vocab=75, width=36, taps=2, eps=1e-6, embed_scale=0.7),
    "wide": config([layer(heads=9, dim=16, rot_dim=8, vdim=24, q_rank=48, kv_rank=144, window=70, ff=96),
                    layer(heads=2, dim=32, rot_dim=16, vdim=8, q_rank=24, kv_rank=264, window=0, mlp="moe", experts=70, top=4,
                          expert_ff=16, shared_ff=32)],
                   vocab=130, width=64, taps=5),
    "one_tap": config([layer(mlp="moe", experts=2, top=1), layer(rot_dim=0, rot_dims=0, scale=0.4)], taps=1, width=24, vocab=50),
}


def checkpoint(cfg_dict, seed=0):
    cfg = fidizen.config_from_dict(cfg_dict)
    return cfg, fidizen.synth_state(cfg, seed=seed)


def build(cfg_dict, dtype, seed=0, page=4, batch=4, max_length=256, max_tokens=1024, sd=None):
    """a served model on cuda:0 over a seeded checkpoint (weights rounded to `dtype`) + the state dict it was built from"""
    cfg = fidizen.config_from_dict(cfg_dict)
    if sd is None:
        sd = fidizen.synth_state(cfg, seed=seed)
    sd = {k: v.to(dtype).to(torch.float32) for k, v in sd.items()}          # the oracle sees exactly the stored weights
    m = fidizen.Fidizen("tiny", batch_size=batch, max_length=max_length, max_tokens=max_tokens, device="cuda:0", dtype=dtype,
                        state_dict=sd, config=cfg, page_size=page)
    m.alloc()
    return m, sd
