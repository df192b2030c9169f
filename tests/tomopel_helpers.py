"""Tiny Tomopel configurations, seeded checkpoints and comparison helpers for the tests of that design."""
import torch

from umbrella_amd.models import tomopel


def parallel(heads=4, kv_heads=2, dim=8, vdim=6, scale=None, bias_max=40, q_temp=(0.3, 8), s_heads=3, s_vdim=4, state=5, groups=1,
             norm_groups=1, conv=3, left_scale=0.7, right_scale=1.2):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale,
            "bias_max": bias_max}
    if q_temp is not None:
        left["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    right = {"heads": s_heads, "vdim": s_vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}
    return "parallel", {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def mingru(width=24):
    return "mingru", {"width": width}


def layer(mixer, mlp="dense", ff=20, experts=5, top=2, expert_ff=12, shared_ff=10):
    if mlp == "dense":
        f = {"kind": "dense", "ff": ff}
    elif mlp == "moe":
        f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff}}
        if shared_ff:
            f["shared"] = {"ff": shared_ff}
    else:
        f = None
    return {"type": mixer[0], "mixer": mixer[1], "mlp": f}


def config(layers, vocab=90, width=40, eps=1e-5, embed_scale=2.0, streams=2, residual_mult=0.8):
    c = {"architecture": "Tomopel", "layers": layers, "norm": {"eps": eps}, "embedding": {"scale": embed_scale}, "vocab": vocab,
         "width": width, "residual_mult": residual_mult}
    if streams is not None:
        c["streams"] = streams
    return c


# shapes that differ from one another in every size: layer order, odd sizes (nothing a multiple of 8), one and three
# streams, as many key/value heads as query heads and one only, groups of B / C, several norm groups, one tap (no
# convolution state) and five, no temperature, all experts used and one of many, no shared expert, no feed-forward,
# a bias table that is exact everywhere a short test reaches and one whose logarithmic part starts at distance 2
CONFIGS = {
    "mixed": config([layer(parallel()), layer(mingru(), mlp="moe"), layer(parallel(heads=2, kv_heads=2, conv=2), mlp="moe", top=1,
                                                                       shared_ff=0, experts=7),
                     layer(mingru(width=17), mlp=None), layer(parallel(s_heads=4, groups=2, norm_groups=2, conv=5), mlp=None)]),
    "odd": config([layer(parallel(heads=3, kv_heads=1, dim=7, vdim=9, s_heads=2, s_vdim=5, state=3, conv=1, q_temp=None, bias_max=9),
                         mlp="moe", experts=3, top=3, expert_ff=5, shared_ff=7),
                   layer(mingru(width=70), ff=17)], vocab=75, width=36, eps=1e-6, embed_scale=0.7, streams=3, residual_mult=1.0),
    "single": config([layer(mingru(width=33), mlp="moe", experts=9, top=4), layer(parallel(heads=6, kv_heads=3, dim=16, vdim=16,
                     s_heads=6, s_vdim=8, state=16, groups=3, norm_groups=3, conv=4, q_temp=(0.5, 1)), ff=48)],
                     vocab=130, width=64, streams=1, residual_mult=0.5),
    "wide": config([layer(parallel(heads=8, kv_heads=2, dim=32, vdim=64, s_heads=4, s_vdim=32, state=64, groups=2, norm_groups=4,
                                   bias_max=300, q_temp=(0.2, 16)), mlp="moe", experts=70, top=4, expert_ff=16, shared_ff=32),
                    layer(mingru(width=300), ff=96)], vocab=110, width=128),
}
BIAS_ROWS = {"mixed": 12, "odd": 4, "single": 7, "wide": 32}


def checkpoint(cfg_dict, seed=0, bias_rows=16, stream_weights=True):
    cfg = tomopel.config_from_dict(cfg_dict)
    sd = tomopel.synth_state(cfg, seed=seed, bias_rows=bias_rows)
    if not stream_weights:
        sd = {k: v for k, v in sd.items() if ".hc" not in k}
    return cfg, sd


def build(cfg_dict, dtype, seed=0, page=4, batch=4, max_length=256, max_tokens=1024, sd=None, bias_rows=16, stream_weights=True):
    """a served model on cuda:0 over a seeded checkpoint (weights rounded to `dtype`) + the state dict it was built from"""
    cfg = tomopel.config_from_dict(cfg_dict)
    if sd is None:
        _, sd = checkpoint(cfg_dict, seed, bias_rows, stream_weights)
    sd = {k: v.to(dtype).to(torch.float32) for k, v in sd.items()}          # the oracle sees exactly the stored weights
    m = tomopel.Tomopel("tiny", batch_size=batch, max_length=max_length, max_tokens=max_tokens, device="cuda:0", dtype=dtype,
                        state_dict=sd, config=cfg, page_size=page)
    m.alloc()
    return m, sd
