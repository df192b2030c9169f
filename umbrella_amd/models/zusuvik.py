"""Zusuvik: a decoder stack whose layers are chosen by the checkpoint's config.json:

* a layer is ``x <- x + (mixer(norm1(x)) + ff(norm2(x)))``: both sublayers read the SAME residual; every norm is an RMS norm
  whose weight is stored around zero (factor ``1 + w``); the head is the embedding table, the logits times a constant;
* ``loop``: a span of layers runs several times in a row with the same weights, each pass with a cache and state of its own;
  before every pass but the first the embedding row joins the residual again;
* ``retention`` -- linear attention with one fixed decay per head, no softmax and no denominator: rotary positions (half
  layout) on q and k, k times dim^-1/2, per-head unit RMS, SiLU gate;
* ``parallel`` -- two mixers reading the same input, their outputs added with two constants: causal softmax attention
  (grouped query heads; q, k, v with biases through a short causal convolution per channel; q / k RMS norm over the whole
  projection; interleaved rotary with frequency scaling of the long wavelengths; scores capped by a tanh) and a matrix memory
  with exponential gates (capped log gates, a running maximum as stabiliser, a normaliser, per-head unit RMS times a weight
  over all heads, sigmoid gate);
* feed-forwards: routed experts chosen by the largest router logits (weights = softmax over the chosen logits, applied to
  the outputs) of the capped gated form ``g sigmoid(1.702 g) (u + 1)``, plus a shared expert of the same form times
  ``sigmoid(w_sg . h)``.

This file only TRANSLATES the design -- config.json keys, tensor names, how matrices are fused or stacked, the loop unrolled
into layers that share tensors -- into the generic sequence-mixer runtime (models/seqmix.py); every mechanism lives there and
in csrc/seq_*.hip with its constants as parameters.
"""
from __future__ import annotations

import json
import os

import torch

from .config import AttnMLSTMCfg, RetentionCfg, SeqLayerCfg, SeqMixCfg
from .seqmix import SeqMixLM

ARCHITECTURE = "Zusuvik"
GLU_ALPHA = 1.702          # the design fixes the sigmoid's factor of its experts


def _rot(m: dict):
    r = m.get("rot") or {}
    return int(r.get("dims", 0)), float(r.get("base", 10000.0)), (dict(r["scaling"]) if r.get("scaling") else None)


def _mixer(kind: str, m: dict):
    if kind == "retention":
        dims, base, scaling = _rot(m)
        return RetentionCfg(heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                            decay=[float(d) for d in m["decay"]], rot_dims=dims, rot_base=base, rot_scaling=scaling,
                            rot_layout="half")
    if kind == "parallel":
        a, b = m["left"], m["right"]
        dims, base, scaling = _rot(a)
        return AttnMLSTMCfg(heads=int(a["heads"]), kv_heads=int(a.get("kv_heads", a["heads"])), dim=int(a["dim"]),
                            vdim=int(a.get("vdim", a["dim"])), scale=float(a["scale"]), softcap=float(a.get("softcap") or 0.0),
                            window=int(a.get("window") or 0), taps=int(a.get("conv") or 1), rot_dims=dims, rot_base=base, rot_scaling=scaling,
                            rot_layout="interleaved", a_scale=float(m.get("left_scale", 1.0)), m_heads=int(b["heads"]),
                            m_dim=int(b["dim"]), m_vdim=int(b.get("vdim", b["dim"])), gate_cap=float(b["gate_cap"]),
                            b_scale=float(m.get("right_scale", 1.0)))
    raise ValueError(f"{ARCHITECTURE}: unknown layer type '{kind}'")


def _layer(entry: dict, index: int) -> SeqLayerCfg:
    mixer = _mixer(entry["type"], entry["mixer"])
    mlp = entry.get("mlp")
    prefix = f"l{index}."
    if mlp is None:
        return SeqLayerCfg(mixer=mixer, ff=0, tensor_prefix=prefix)
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"{ARCHITECTURE}: unknown feed-forward kind '{mlp.get('kind')}'")
    shared = mlp.get("shared")
    return SeqLayerCfg(mixer=mixer, ff=0, ff_kind="moe", experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                       expert_ff=int(mlp["expert"]["ff"]), shared_ff=int(shared["ff"]) if shared else 0, act="clamp_glu",
                       route="top_logits", act_limit=float(mlp["expert"]["limit"]),
                       shared_limit=float(shared["limit"]) if shared else 0.0, act_alpha=GLU_ALPHA, shared_gate=bool(shared),
                       tensor_prefix=prefix)


def layer_runs(n_layers: int, loop: dict | None):
    """the order the layers run in: [(layer index, starts a repeated pass)]; layers start .. stop - 1 run ``times`` times in a row"""
    lp = loop or {}
    start, stop, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
    if not (0 <= start < stop <= n_layers) or times <= 1:
        return [(i, False) for i in range(n_layers)]
    runs = [(i, False) for i in range(start)]
    for p in range(times):
        runs += [(i, p > 0 and i == start) for i in range(start, stop)]
    return runs + [(i, False) for i in range(stop, n_layers)]


def config_from_dict(c: dict, name: str = "zusuvik") -> SeqMixCfg:
    """config.json -> the runtime's layer list: the loop is unrolled, a repeated layer uses the tensors of its first run
    (``weights_of``) with a cache and state of its own, and the first layer of every further pass adds the embedding row"""
    layers, first_run = [], {}
    for i, again in layer_runs(len(c["layers"]), c.get("loop")):
        ly = _layer(c["layers"][i], i)
        if i in first_run:
            ly.weights_of = first_run[i]
        else:
            first_run[i] = len(layers)
        ly.add_embed = again
        layers.append(ly)
    return SeqMixCfg(vocab_size=int(c["vocab"]), width=int(c["width"]), norm_eps=float(c["norm"]["eps"]), norm_groups=1,
                     layers=layers, name=name, architecture=ARCHITECTURE, norm_offset=1.0, block="parallel",
                     logit_scale=float(c.get("logit_scale", 1.0)))


def config_from_dir(path: str) -> SeqMixCfg:
    with open(os.path.join(path, "config.json")) as f:
        return config_from_dict(json.load(f), name=os.path.basename(os.path.normpath(path)))


def tensor_shapes(cfg: SeqMixCfg) -> dict:
    """checkpoint tensor name -> shape (linear weights are [out, in])"""
    W = cfg.width
    sh = {"embed": (cfg.vocab_size, W), "final.norm": (W,)}
    for ly in cfg.layers:
        if ly.weights_of is not None:
            continue
        p, m = ly.tensor_prefix, ly.mixer
        sh[p + "norm1"] = (W,)
        if m.kind == "retention":
            sh.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W), p + "mix.v": (m.heads * m.vdim, W),
                       p + "mix.g": (m.heads * m.vdim, W), p + "mix.o": (W, m.heads * m.vdim)})
        else:
            a, b = p + "mix.left.", p + "mix.right."
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            sh.update({a + "q": (nq, W), a + "q.b": (nq,), a + "k": (nk, W), a + "k.b": (nk,), a + "v": (nv, W), a + "v.b": (nv,),
                       a + "q.norm": (nq,), a + "k.norm": (nk,), a + "q.conv": (nq, m.taps), a + "k.conv": (nk, m.taps),
                       a + "v.conv": (nv, m.taps), a + "o": (W, m.heads * m.vdim), a + "o.b": (W,),
                       b + "q": (m.m_heads * m.m_dim, W), b + "k": (m.m_heads * m.m_dim, W), b + "v": (m.m_heads * m.m_vdim, W),
                       b + "g": (m.m_heads * m.m_vdim, W), b + "o": (W, m.m_heads * m.m_vdim), b + "norm": (m.m_heads * m.m_vdim,),
                       b + "i": (m.m_heads, W), b + "i.b": (m.m_heads,), b + "f": (m.m_heads, W), b + "f.b": (m.m_heads,)})
        if not ly.has_ff:
            continue
        sh[p + "norm2"] = (W,)
        sh.update({p + "mlp.router": (ly.experts, W), p + "mlp.router.b": (ly.experts,)})
        for e in [f"e{k}" for k in range(ly.experts)] + (["shared"] if ly.shared_ff else []):
            f = ly.shared_ff if e == "shared" else ly.expert_ff
            sh.update({p + f"mlp.{e}.gate": (f, W), p + f"mlp.{e}.up": (f, W), p + f"mlp.{e}.down": (W, f)})
        if ly.shared_ff:
            sh[p + "mlp.shared.sg"] = (1, W)
    return sh


def synth_state(cfg: SeqMixCfg, seed: int = 0) -> dict:
    """Seeded random fp32 checkpoint of the design (tests, benchmarks): name -> tensor."""
    g = torch.Generator().manual_seed(seed)
    sd = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".", 1)[-1] if name[0] == "l" and name[1].isdigit() else name
        r = lambda: torch.randn(shape, generator=g)                     # noqa: E731
        if leaf in ("norm1", "norm2", "final.norm"):
            t = 0.1 * r()                                               # stored around zero
        elif leaf.endswith(".norm"):
            t = 1.0 + 0.1 * r()
        elif leaf == "embed":
            t = r()
        elif leaf.endswith(".conv"):
            t = 0.6 * r()
        elif leaf.endswith(".b"):
            t = 0.5 * r()
        elif leaf in ("mix.right.i", "mix.right.f", "mlp.router"):
            t = 2.0 * r() / shape[1] ** 0.5
        else:
            t = r() / shape[1] ** 0.5
        sd[name] = t
    return sd


class Zusuvik(SeqMixLM):
    """``AutoModelLM`` resolves a directory whose config.json says ``"architecture": "Zusuvik"`` to this class."""

    @staticmethod
    def read_config(path: str) -> SeqMixCfg:
        return config_from_dir(path)

    def layer_tensors(self, i: int, ly: SeqLayerCfg, get):
        """The design's tensor names -> the runtime's fused per-layer tensors.  ``get(name)`` fetches one checkpoint tensor
        in the storage dtype on the device."""
        p, m = ly.tensor_prefix or f"l{i}.", ly.mixer
        t = {"norm1": get(p + "norm1"), "norm1b": None}
        if m.kind == "retention":
            t["proj_w"] = torch.cat([get(p + "mix.q"), get(p + "mix.k"), get(p + "mix.v"), get(p + "mix.g")], dim=0)
            t["out_w"] = get(p + "mix.o")
            assert t["proj_w"].shape[0] == 2 * m.heads * (m.dim + m.vdim) and t["out_w"].shape[1] == m.heads * m.vdim
        else:
            a, b = p + "mix.left.", p + "mix.right."
            ws = [get(a + "q"), get(a + "k"), get(a + "v"), get(b + "q"), get(b + "k"), get(b + "v"), get(b + "g"), get(b + "i"),
                  get(b + "f")]
            bs = [get(a + "q.b"), get(a + "k.b"), get(a + "v.b")] + [torch.zeros_like(w[:, 0]) for w in ws[3:7]] + \
                 [get(b + "i.b"), get(b + "f.b")]
            t["proj_w"], t["proj_b"] = torch.cat(ws, dim=0), torch.cat(bs)          # ONE input projection for both mixers
            # ONE output projection over [a_scale * attention | b_scale * memory]; the attention's output bias with its constant
            t["out_w"] = torch.cat([get(a + "o"), get(b + "o")], dim=1).contiguous()
            t["out_b"] = (get(a + "o.b").to(torch.float32) * m.a_scale).to(self.dtype)
            t["q_norm"], t["k_norm"], t["m_norm"] = get(a + "q.norm"), get(a + "k.norm"), get(b + "norm")
            t["c_conv"] = torch.cat([get(a + "q.conv"), get(a + "k.conv"), get(a + "v.conv")], dim=0)
            C = (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim
            assert tuple(t["c_conv"].shape) == (C, m.taps), tuple(t["c_conv"].shape)
            assert t["proj_w"].shape[0] == C + 2 * m.m_heads * (m.m_dim + m.m_vdim) + 2 * m.m_heads
            assert t["q_norm"].numel() == m.heads * m.dim and t["k_norm"].numel() == m.kv_heads * m.dim
        if not ly.has_ff:
            return t
        t["norm2"], t["norm2b"] = get(p + "norm2"), None
        rw, rb = get(p + "mlp.router"), get(p + "mlp.router.b")
        names = [f"mlp.e{k}" for k in range(ly.experts)]
        t["e_gu"] = torch.stack([torch.cat([get(p + n + ".gate"), get(p + n + ".up")], dim=0) for n in names])   # [E][2F][W]
        t["e_down"] = torch.stack([get(p + n + ".down") for n in names])                                         # [E][W][F]
        if ly.shared_ff:
            # the shared expert's gate is one more row of the router's product
            rw, rb = torch.cat([rw, get(p + "mlp.shared.sg").reshape(1, -1)], dim=0), torch.cat([rb, torch.zeros_like(rb[:1])])
            t["s_gu_w"] = torch.cat([get(p + "mlp.shared.gate"), get(p + "mlp.shared.up")], dim=0)
            t["s_down_w"] = get(p + "mlp.shared.down")
        t["router_w"], t["router_b"] = rw, rb
        return t

    def top_tensors(self, get):
        embed = get("embed")
        return {"embed": embed, "final_norm": get("final.norm"), "head": embed}          # the head is the embedding table
