"""Tomopel: a decoder stack over SEVERAL residual streams whose layers are chosen by the checkpoint's config.json:

* the residual is ``streams`` copies per token; a sublayer reads ``sum_s in[s] x_s`` through an RMS norm whose weight is
  stored around zero (factor ``1 + w``) and writes back ``x_t <- sum_s mix[s, t] x_s + m out[t] y`` (``m`` =
  ``residual_mult``); the model ends with the same norm of the sum of the streams; the embedding is scaled by a constant;
* ``mingru`` -- a minimal gated recurrence: gates from the current token only, one fp32 state per channel, SiLU output gate;
* ``parallel`` -- two mixers reading the same input, their outputs added with two constants: causal softmax attention
  (grouped query heads, unit-RMS q / k with a shared weight, weightless unit-RMS values, a query temperature that grows with
  the logarithm of the position, a learned bias per (distance bucket, head): exact buckets below half the table, logarithmic
  ones up to ``bias_max``, one sigmoid gate per head) and a state-space layer with one decay per head (input convolution,
  softplus step sizes, ``[state, vdim]`` fp32 state per head, skip term, gated RMS norm in groups);
* feed-forwards: dense gated SiLU, or routed experts with softmax scores (chosen by score + correction, weights renormalised
  over the chosen, applied to the experts' outputs), experts and the always-on shared expert of the form
  ``W_down relu(W_up h)^2``.

This file only TRANSLATES the design -- config.json keys, tensor names, how matrices are fused or stacked, the bucket
function expanded into a bias-by-distance table -- into the generic sequence-mixer runtime (models/seqmix.py); every
mechanism lives there and in csrc/seq_*.hip with its constants as parameters.
"""
from __future__ import annotations

import json
import math
import os

import torch

from .config import AttnSSDCfg, MinGRUCfg, SeqLayerCfg, SeqMixCfg
from .seqmix import SeqMixLM

ARCHITECTURE = "Tomopel"


def _mixer(kind: str, m: dict):
    if kind == "mingru":
        return MinGRUCfg(dim=int(m["width"]))
    if kind == "parallel":
        a, b = m["left"], m["right"]
        qt = a.get("q_temp") or {}
        return AttnSSDCfg(heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", a["heads"])), dim=int(a["dim"]),
                          vdim=int(a.get("vdim", a["dim"])), scale=float(a["scale"]), window=int(a.get("window", 0)),
                          bias_rows=0, bias_far=float(a.get("bias_max", 0)), temp_coef=float(qt.get("coef", 0.0)),
                          temp_every=int(qt.get("every", 0)), a_scale=float(m.get("left_scale", 1.0)),
                          s_heads=int(b["heads"]), s_vdim=int(b["vdim"]), s_state=int(b["state"]), s_groups=int(b.get("groups", 1)),
                          s_norm_groups=int(b.get("norm_groups", 1)), s_taps=int(b.get("conv", 1)),
                          b_scale=float(m.get("right_scale", 1.0)))
    raise ValueError(f"{ARCHITECTURE}: unknown layer type '{kind}'")


def _layer(entry: dict) -> SeqLayerCfg:
    mixer = _mixer(entry["type"], entry["mixer"])
    mlp = entry.get("mlp")
    if mlp is None:
        return SeqLayerCfg(mixer=mixer, ff=0)
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return SeqLayerCfg(mixer=mixer, ff=int(mlp["ff"]), ff_kind="gated")
    if kind == "moe":
        shared = mlp.get("shared")
        return SeqLayerCfg(mixer=mixer, ff=0, ff_kind="moe", experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                           expert_ff=int(mlp["expert"]["ff"]), shared_ff=int(shared["ff"]) if shared else 0, act="relu2",
                           route="softmax_out")
    raise ValueError(f"{ARCHITECTURE}: unknown feed-forward kind '{kind}'")


def config_from_dict(c: dict, name: str = "tomopel") -> SeqMixCfg:
    return SeqMixCfg(vocab_size=int(c["vocab"]), width=int(c["width"]), norm_eps=float(c["norm"]["eps"]), norm_groups=1,
                     layers=[_layer(e) for e in c["layers"]], name=name, architecture=ARCHITECTURE,
                     embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)), streams=int(c.get("streams", 1)),
                     resid_mult=float(c.get("residual_mult", 1.0)), norm_offset=1.0)


def config_from_dir(path: str) -> SeqMixCfg:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))


def distance_buckets(rows: int, far: float, n: int) -> torch.Tensor:
    """bucket of every distance 0 .. n - 1 (int64): the distance itself below rows // 2, then logarithmic steps that reach
    the last row at distance ``far``; fp32 arithmetic"""
    d = torch.arange(n, dtype=torch.int64)
    half = rows // 2
    if half < 1 or not far > half:
        return torch.where(d < half, d, torch.full_like(d, rows - 1))
    steps = torch.log(d.clamp_min(1).to(torch.float32) / half) / math.log(far / half) * (rows - half)
    large = (half + steps.floor().to(torch.int64)).clamp(max=rows - 1)
    return torch.where(d < half, d, large)


def bias_by_distance(rel: torch.Tensor, far: float, max_len: int) -> torch.Tensor:
    """the learned table [rows, heads] -> fp32 [heads, n_dist] indexed by the distance itself; distances from n_dist - 1 on
    share the last entry (every distance the table tells apart, or every distance a sequence of max_len can hold)"""
    rows = rel.shape[0]
    n = int(max(1, min(max_len, max(math.ceil(far), rows // 2) + 1)))
    b = distance_buckets(rows, far, n)
    last = int((b == rows - 1).nonzero()[0]) if bool((b == rows - 1).any()) else n - 1
    return rel.to(torch.float32)[b[:last + 1].to(rel.device)].t().contiguous()


def tensor_shapes(cfg: SeqMixCfg, bias_rows: int = 16) -> dict:
    """checkpoint tensor name -> shape (linear weights are [out, in])"""
    W, S = cfg.width, cfg.streams
    sh = {"embed": (cfg.vocab_size, W), "final.norm": (W,), "head": (cfg.vocab_size, W)}
    for i, ly in enumerate(cfg.layers):
        p, m = f"l{i}.", ly.mixer
        sh[p + "norm1"] = (W,)
        for q in ("hc1", "hc2") if ly.has_ff else ("hc1",):
            sh.update({p + q + ".in": (S,), p + q + ".out": (S,), p + q + ".mix": (S, S)})
        if m.kind == "mingru":
            sh.update({p + "mix.z": (m.dim, W), p + "mix.z.b": (m.dim,), p + "mix.x": (m.dim, W), p + "mix.x.b": (m.dim,),
                       p + "mix.g": (m.dim, W), p + "mix.o": (W, m.dim)})
        else:
            inner, gn = m.s_heads * m.s_vdim, m.s_groups * m.s_state
            sh.update({p + "mix.left.q": (m.heads * m.dim, W), p + "mix.left.k": (m.kv_heads * m.dim, W),
                       p + "mix.left.v": (m.kv_heads * m.vdim, W), p + "mix.left.q.norm": (m.dim,), p + "mix.left.k.norm": (m.dim,),
                       p + "mix.left.rel": (m.bias_rows or bias_rows, m.heads), p + "mix.left.g": (m.heads, W),
                       p + "mix.left.o": (W, m.heads * m.vdim),
                       p + "mix.right.in": (2 * inner + 2 * gn + m.s_heads, W), p + "mix.right.conv": (inner + 2 * gn, m.s_taps),
                       p + "mix.right.conv.b": (inner + 2 * gn,), p + "mix.right.dt_bias": (m.s_heads,),
                       p + "mix.right.A_log": (m.s_heads,), p + "mix.right.D": (m.s_heads,), p + "mix.right.norm": (inner,),
                       p + "mix.right.o": (W, inner)})
        if not ly.has_ff:
            continue
        sh[p + "norm2"] = (W,)
        if ly.ff_kind == "gated":
            sh.update({p + "mlp.gate": (ly.ff, W), p + "mlp.up": (ly.ff, W), p + "mlp.down": (W, ly.ff)})
        else:
            sh.update({p + "mlp.router": (ly.experts, W), p + "mlp.correction": (ly.experts,)})
            for e in [f"e{k}" for k in range(ly.experts)] + (["shared"] if ly.shared_ff else []):
                f = ly.shared_ff if e == "shared" else ly.expert_ff
                sh.update({p + f"mlp.{e}.up": (f, W), p + f"mlp.{e}.down": (W, f)})
    return sh


def synth_state(cfg: SeqMixCfg, seed: int = 0, bias_rows: int = 16) -> dict:
    """Seeded random fp32 checkpoint of the design (tests, benchmarks): name -> tensor."""
    g = torch.Generator().manual_seed(seed)
    sd, S = {}, cfg.streams
    for name, shape in tensor_shapes(cfg, bias_rows).items():
        leaf = name.split(".", 1)[-1] if name[0] == "l" and name[1].isdigit() else name
        r = lambda: torch.randn(shape, generator=g)                     # noqa: E731
        if leaf in ("norm1", "norm2", "final.norm"):
            t = 0.1 * r()                                               # stored around zero
        elif leaf in ("mix.left.q.norm", "mix.left.k.norm", "mix.right.norm"):
            t = 1.0 + 0.1 * r()
        elif leaf == "embed":
            t = r()
        elif leaf.endswith(".in"):
            t = 1.0 / S + 0.2 * r()
        elif leaf.endswith(".out"):
            t = 1.0 + 0.2 * r()
        elif leaf.endswith(".mix"):
            t = torch.eye(S) + 0.2 * r()
        elif leaf == "mix.left.rel":
            t = 0.7 * r()
        elif leaf in ("mix.z.b", "mix.x.b", "mix.right.conv.b"):
            t = 0.3 * r()
        elif leaf == "mix.right.conv":
            t = 0.5 * r()
        elif leaf == "mix.right.dt_bias":
            t = -1.0 + 0.5 * r()
        elif leaf == "mix.right.A_log":
            t = 0.5 * r()
        elif leaf == "mix.right.D":
            t = 1.0 + 0.2 * r()
        elif leaf == "mlp.correction":
            t = 0.05 * r()
        elif leaf == "mlp.router":
            t = 2.0 * r() / shape[1] ** 0.5
        else:
            t = r() / shape[1] ** 0.5
        sd[name] = t
    return sd


class Tomopel(SeqMixLM):
    """``AutoModelLM`` resolves a directory whose config.json says ``"architecture": "Tomopel"`` to this class."""

    @staticmethod
    def read_config(path: str) -> SeqMixCfg:
        return config_from_dir(path)

    def _streams(self, t: dict, p: str, q: str, get, has):
        """read / write / mix weights of one sublayer, fp32; a checkpoint without them has the plain residual"""
        for part in ("in", "out", "mix"):
            name = f"{p}{q}.{part}"
            t[f"{q}_{part}"] = get(name).to(torch.float32).contiguous() if has(name) else None

    def layer_tensors(self, i: int, ly: SeqLayerCfg, get):
        """The design's tensor names -> the runtime's fused per-layer tensors.  ``get(name)`` fetches one checkpoint
        tensor in the storage dtype on the device."""
        p, m = f"l{i}.", ly.mixer
        has = self.has_tensor
        f32 = lambda name: get(name).to(torch.float32).contiguous()      # noqa: E731
        t = {"norm1": get(p + "norm1"), "norm1b": None}
        self._streams(t, p, "hc1", get, has)
        if m.kind == "mingru":
            zb, xb = get(p + "mix.z.b"), get(p + "mix.x.b")
            t["proj_w"] = torch.cat([get(p + "mix.z"), get(p + "mix.x"), get(p + "mix.g")], dim=0)           # [z | x | g]
            t["proj_b"] = torch.cat([zb, xb, torch.zeros_like(zb)])
            t["out_w"] = get(p + "mix.o")
            assert t["proj_w"].shape[0] == 3 * m.dim and t["out_w"].shape[1] == m.dim
        else:
            a, b = p + "mix.left.", p + "mix.right."
            t["proj_w"] = torch.cat([get(a + "q"), get(a + "k"), get(a + "v"), get(a + "g"), get(b + "in")], dim=0)
            t["out_w"] = torch.cat([get(a + "o"), get(b + "o")], dim=1).contiguous()                          # over [left | right]
            t["q_norm"], t["k_norm"] = get(a + "q.norm"), get(a + "k.norm")
            if has(a + "rel"):
                rel = f32(a + "rel")
                m.bias_rows = rel.shape[0]
                t["dist_bias"] = bias_by_distance(rel, m.bias_far, self.max_length)
            t["s_conv"], t["s_conv_b"], t["s_norm"] = get(b + "conv"), get(b + "conv.b"), get(b + "norm")
            t["s_dt_bias"], t["s_a_log"], t["s_d"] = f32(b + "dt_bias"), f32(b + "A_log"), f32(b + "D")
            inner, gn = m.s_heads * m.s_vdim, m.s_groups * m.s_state
            assert t["proj_w"].shape[0] == m.heads * m.dim + m.kv_heads * (m.dim + m.vdim) + m.heads + 2 * inner + 2 * gn + m.s_heads
            assert tuple(t["s_conv"].shape) == (inner + 2 * gn, m.s_taps)
        if not ly.has_ff:
            return t
        t["norm2"], t["norm2b"] = get(p + "norm2"), None
        self._streams(t, p, "hc2", get, has)
        if ly.ff_kind == "gated":
            t["gu_w"], t["down_w"] = torch.cat([get(p + "mlp.gate"), get(p + "mlp.up")], dim=0), get(p + "mlp.down")
        else:
            t["router_w"] = get(p + "mlp.router")
            t["correction"] = f32(p + "mlp.correction") if has(p + "mlp.correction") else None
            names = [f"mlp.e{k}" for k in range(ly.experts)]
            t["e_gu"] = torch.stack([get(p + n + ".up") for n in names])             # [E][F][W]: no gate, the up-projection alone
            t["e_down"] = torch.stack([get(p + n + ".down") for n in names])         # [E][W][F]
            if ly.shared_ff:
                t["s_gu_w"], t["s_down_w"] = get(p + "mlp.shared.up"), get(p + "mlp.shared.down")
        return t

    def top_tensors(self, get):
        return {"embed": get("embed"), "final_norm": get("final.norm"), "head": get("head")}
