"""Tiny Zusuvik configurations, seeded checkpoints and comparison helpers for the tests of that design."""
import torch

from umbrella_amd.models import zusuvik

SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}


def retention(heads=3, dim=8, vdim=6, decay=(0.9, 0.97, 0.995), rot_dims=8, base=100.0):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot_dims:
        m["rot"] = {"base": base, "dims": rot_dims}
    return "retention", m


def parallel(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, rot_dims=4, base=50.0, scaling=SCALING, scale=None, softcap=5.0,
             m_heads=3, m_dim=5, m_vdim=7, gate_cap=6.0, left_scale=0.7, right_scale=1.2):
    rot = {"base": base, "dims": rot_dims}
    if scaling:
        rot["scaling"] = dict(scaling)
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "rot": rot,
            "scale": dim ** -0.5 if scale is None else scale, "softcap": softcap}
    right = {"heads": m_heads, "dim": m_dim, "vdim": m_vdim, "gate_cap": gate_cap}
    return "parallel", {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


def layer(mixer, mlp="moe", experts=5, top=2, expert_ff=12, limit=1.5, shared_ff=10, shared_limit=1.0):
    f = None
    if mlp == "moe":
        f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": expert_ff, "limit": limit}}
        if shared_ff:
            f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return {"type": mixer[0], "mixer": mixer[1], "mlp": f}


def config(layers, vocab=90, width=40, eps=1e-5, logit_scale=1.5, loop=None):
    c = {"architecture": "Zusuvik", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width, "logit_scale": logit_scale}
    if loop:
        c["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return c


# shapes that differ from one another in every size: layer order, odd sizes (nothing a multiple of 8), a loop in the middle run
# three times / over everything / none, as many key/value heads as query heads and one only, one tap (no convolution state) and
# four, rotary on all / some / none of the features, scaled frequencies or not, a decay of exactly 1, all experts used and one of
# many, no shared expert, no feed-forward, a logit scale of 1
CONFIGS = {
    "mixed": config([layer(retention()), layer(parallel()), layer(retention(heads=2, dim=6, vdim=9, decay=(1.0, 0.5), rot_dims=4),
                                                                  top=1, shared_ff=0, experts=7),
                     layer(parallel(heads=2, kv_heads=2, conv=2, scaling=None, softcap=30.0), mlp=None)], loop=(1, 3, 3)),
    "odd": config([layer(parallel(heads=3, kv_heads=1, dim=7, vdim=9, conv=1, rot_dims=6, m_heads=2, m_dim=3, m_vdim=3), experts=3, top=3,
                         expert_ff=5, shared_ff=7, limit=0.7, shared_limit=2.5),
                   layer(retention(heads=1, dim=5, vdim=3, decay=(0.93,), rot_dims=0), mlp=None)], vocab=75, width=36, eps=1e-6,
                  logit_scale=1.0, loop=(0, 2, 2)),
    "plain": config([layer(retention(heads=4, dim=16, vdim=16, decay=(0.9, 0.95, 0.99, 0.999), rot_dims=16)),
                     layer(parallel(heads=6, kv_heads=3, dim=16, vdim=16, conv=4, rot_dims=16, m_heads=2, m_dim=16, m_vdim=12),
                           experts=9, top=4)], vocab=130, width=64, logit_scale=0.5),
    "wide": config([layer(parallel(heads=8, kv_heads=2, dim=32, vdim=64, rot_dims=8, m_heads=4, m_dim=32, m_vdim=48), experts=70, top=4,
                          expert_ff=16, shared_ff=32),
                    layer(retention(heads=4, dim=64, vdim=32, decay=(0.98, 0.99, 0.995, 0.999), rot_dims=32, base=10000.0))],
                   vocab=110, width=128, loop=(0, 1, 2)),
}


def checkpoint(cfg_dict, seed=0):
    cfg = zusuvik.config_from_dict(cfg_dict)
    return cfg, zusuvik.synth_state(cfg, seed=seed)


def build(cfg_dict, dtype, seed=0, page=4, batch=4, max_length=256, max_tokens=1024, sd=None, **kw):
    """a served model on cuda:0 over a seeded checkpoint (weights rounded to `dtype`) + the state dict it was built from"""
    cfg = zusuvik.config_from_dict(cfg_dict)
    if sd is None:
        _, sd = checkpoint(cfg_dict, seed)
    sd = {k: v.to(dtype).to(torch.float32) for k, v in sd.items()}          # the oracle sees exactly the stored weights
    m = zusuvik.Zusuvik("tiny", batch_size=batch, max_length=max_length, max_tokens=max_tokens, device="cuda:0", dtype=dtype,
                        state_dict=sd, config=cfg, page_size=page, **kw)
    m.alloc()
    return m, sd
