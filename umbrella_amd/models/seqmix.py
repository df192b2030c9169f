"""Runtime of the sequence-mixer model family on the HIP path (libumbrella_seq.so, include/umbrella_seq.h).

A model is a LIST of layers, each a token mixer -- windowed attention with pooled blocks, gated linear attention, latent
attention, a minimal gated recurrence, softmax attention beside a state-space layer, retention, or convolved softmax
attention beside a matrix memory -- plus an optional feed-forward (gated SiLU, PolyNorm, or routed experts with a shared one).  A sublayer reads either a grouped RMS norm of the residual stream or the
stream itself through a short causal convolution; its output is normed before it is added back; or (``streams >= 1``) the
residual is several streams that every sublayer reads as one combination and writes back to all.  A layer may use another
layer's tensors with a cache and state of its own; or (``block == "parallel"``) both sublayers of a layer read the same
residual and their outputs are added to it together.  The list, every size and every
constant come from a ``SeqMixCfg`` (models/config.py); a design contributes a subclass that names its checkpoint tensors
(models/gitopel.py, models/fidizen.py).

Unlike the tree-decoding ``Llama`` runtime this one serves MANY sequences: a step is a ragged batch (the rows of each
sequence contiguous, nothing padded), key/value pages and recurrent-state slots are handed out by
``attn.cache.PagedSeqCache``, and the residual stream is fp32.  ``dtype`` may be bfloat16 / float16 (weights, cached
keys, matrix-product inputs in 16 bits; norms, scores, decays, state and accumulators in fp32) or float32 (everything).

Everything numeric runs in the library; this class owns buffers and descriptors.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

from .. import _lib
from .._lib import UmbSeqLayer, UmbSeqLinear, UmbSeqModel, UmbSeqStep, UmbSeqWork
from ..attn.cache import PagedSeqCache
from .base import LLMBase
from .config import SeqMixCfg, rotary_frequencies

KIND_CODE = {"attention": 0, "gla": 1, "latent_attention": 2, "mingru": 3, "attention_ssd": 4, "retention": 5,
             "attention_mlstm": 6}
FF_CODE = {"gated": 0, "polynorm": 1, "moe": 2}
ACT_CODE = {"silu_gated": 0, "relu2": 1, "clamp_glu": 2}
ROUTE_CODE = {"sigmoid_in": 0, "softmax_out": 1, "top_logits": 2}
BLOCK_CODE = {"sequential": 0, "parallel": 1}
ROT_LAYOUT_CODE = {"half": 0, "interleaved": 1}


def _linear(w, b=None) -> UmbSeqLinear:
    s = UmbSeqLinear()
    s.w, s.bias = w.data_ptr(), (b.data_ptr() if b is not None else None)
    s.N, s.K = w.shape
    return s


class SeqMixLM(LLMBase):
    """Subclasses provide ``read_config(path)``, ``layer_tensors(i, layer_cfg, get)`` and ``top_tensors(get)``."""

    def __init__(self, model_name: str, batch_size: int = 1, max_length: int = 256, device: str = "cuda:0",
                 dtype=torch.bfloat16, offload: bool = False, cuda_graph: bool = False, state_dict=None,
                 config: SeqMixCfg | None = None, seed: int = 0, max_tokens: int | None = None, page_size: int = 64,
                 max_step_tokens: int | None = None, hip_graph: bool | None = None) -> None:
        super().__init__()
        if offload:
            raise ValueError("sequence-mixer models are device resident (offload is not supported)")
        self.model_name, self.device, self.dtype = model_name, device, dtype
        self.batch_size = max(1, int(batch_size))              # sequence slots
        self.max_length = int(max_length)                      # longest sequence
        self.max_tokens = int(max_tokens) if max_tokens else self.batch_size * self.max_length   # tokens held by all
        self.page_size = int(page_size)
        self.max_step_tokens = int(max_step_tokens) if max_step_tokens else None
        self._state, self._seed = state_dict, seed
        # hip_graph=True (or UMB_SEQ_GRAPH=1): decode steps (one token per sequence) replay a hipGraph captured per batch
        # size -- ~70 launches become one; the step's indices live in a static device buffer that is rewritten before every
        # replay.  Off by default: a decode step of these models is bound by its kernels, not by launches (1b-class shape,
        # batch 1: 0.59 ms replayed against 0.55 ms launched eagerly).
        self.use_graph = (os.environ.get("UMB_SEQ_GRAPH", "0") == "1") if hip_graph is None else bool(hip_graph)
        self._graphs = {}
        if config is not None:
            self.config = config
        elif os.path.isdir(str(model_name)):
            self.config = self.read_config(model_name)
        else:
            raise ValueError(f"'{model_name}' is not a model directory and no config was given")
        self.eos_tokens = list(self.config.eos_token_id)
        self.ws_tokens = self.logit_rows = 0

    # ------------------------------------------------------------------ weights
    def _getter(self):
        dev, dt = self.device, self.dtype
        if self._state is not None:
            sd = self._state
            self._names = set(sd.keys())
            return lambda name: sd[name].to(device=dev, dtype=dt if sd[name].is_floating_point() else None).contiguous()
        from safetensors import safe_open
        files = [os.path.join(self.model_name, f) for f in sorted(os.listdir(self.model_name)) if f.endswith(".safetensors")]
        index = {}
        for f in files:
            with safe_open(f, "pt") as h:
                for k in h.keys():
                    index[k] = f
        self._names = set(index.keys())

        def get(name):
            with safe_open(index[name], "pt") as h:
                t = h.get_tensor(name)
            return t.to(device=dev, dtype=dt if t.is_floating_point() else None).contiguous()
        return get

    def has_tensor(self, name: str) -> bool:
        """whether the checkpoint holds a tensor of that name (valid while ``alloc`` reads the weights)"""
        return name in self._names

    def alloc(self, **kwargs):
        c, dev, dt = self.config, self.device, self.dtype
        _lib.load_seq()
        get = self._getter()
        self._top = self.top_tensors(get)
        assert tuple(self._top["embed"].shape) == (c.vocab_size, c.width), tuple(self._top["embed"].shape)
        L = len(c.layers)
        self._tensors, kv_layers, state_layers, latent_layers, n_conv, mixer_convs = [], [], [], [], 0, []
        for i, ly in enumerate(c.layers):
            if ly.weights_of is not None:
                # the tensors of another layer (which must own its tensors), a cache and state of this layer's own
                if not (0 <= ly.weights_of < i) or c.layers[ly.weights_of].weights_of is not None:
                    raise ValueError(f"layer {i}: weights_of must name an earlier layer that has tensors of its own")
                t = dict(self._tensors[ly.weights_of])
            else:
                t = self.layer_tensors(i, ly, get)
                t = {k: (v.contiguous() if isinstance(v, torch.Tensor) else v) for k, v in t.items()}
            m = ly.mixer
            if m.kind == "attention":
                if m.vdim != m.dim:
                    raise ValueError("values are the key projection: vdim must equal dim")
                if m.heads % m.kv_heads:
                    raise ValueError("heads must be a multiple of kv_heads")
                t["cache_index"] = len(kv_layers)
                kv_layers.append((m.kv_heads, m.dim, m.pool))
            elif m.kind == "latent_attention":
                t["cache_index"] = len(latent_layers)
                latent_layers.append(m.kv_rank + m.rot_dim)
            elif m.kind == "mingru":
                t["cache_index"] = len(state_layers)
                state_layers.append((1, 1, m.dim))
            elif m.kind == "attention_ssd":
                if m.heads % m.kv_heads or m.s_heads % m.s_groups or (m.s_heads * m.s_vdim) % m.s_norm_groups:
                    raise ValueError("heads / kv_heads, state-space heads / groups and inner width / norm groups must divide")
                t["cache_index"], t["state_index"], t["mconv_index"] = len(kv_layers), len(state_layers), len(mixer_convs)
                kv_layers.append((m.kv_heads, m.dim, 0, m.vdim))
                state_layers.append((m.s_heads, m.s_state, m.s_vdim))
                mixer_convs.append((m.s_taps, m.s_heads * m.s_vdim + 2 * m.s_groups * m.s_state))
            elif m.kind == "retention":
                if len(m.decay) != m.heads:
                    raise ValueError("retention wants one decay per head")
                t["cache_index"] = len(state_layers)
                state_layers.append((m.heads, m.dim, m.vdim))
                t["decay"] = torch.tensor([float(d) for d in m.decay], dtype=torch.float32, device=dev)
            elif m.kind == "attention_mlstm":
                if m.heads % m.kv_heads:
                    raise ValueError("heads must be a multiple of kv_heads")
                t["cache_index"], t["state_index"], t["mconv_index"] = len(kv_layers), len(state_layers), len(mixer_convs)
                kv_layers.append((m.kv_heads, m.dim, 0, m.vdim))
                state_layers.append((m.m_heads, m.m_dim, m.m_pad))      # value column m_vdim carries the normaliser
                state_layers.append((m.m_heads, 1, 1))                  # the running maximum
                mixer_convs.append((m.taps, (m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim))
            else:
                t["cache_index"] = len(state_layers)
                state_layers.append((m.heads, m.dim, m.vdim))
            if m.kind in ("attention", "latent_attention") and "rot_freq" not in t:
                i2 = torch.arange(m.rot_dims // 2, dtype=torch.float32)
                t["rot_freq"] = (m.rot_base ** (-2 * i2 / m.rot_dims)).to(dev) if m.rot_dims else None     # fp32 frequencies
            if m.kind in ("retention", "attention_mlstm") and "rot_freq" not in t:
                t["rot_freq"] = rotary_frequencies(m.rot_base, m.rot_dims, m.rot_scaling).to(dev) if m.rot_dims else None
            if c.canon_taps > 0:
                t["conv_index"] = n_conv
                n_conv += 2 if ly.has_ff else 1
            self._tensors.append(t)
        self.kv_cache = PagedSeqCache(kv_layers, state_layers, self.max_tokens, self.batch_size, dev, dt, page=self.page_size,
                                      latent_layers=latent_layers, conv_states=n_conv, conv_taps=c.canon_taps, width=c.width,
                                      mixer_convs=mixer_convs)
        self._layer_structs = (UmbSeqLayer * L)()
        for i, (ly, t) in enumerate(zip(c.layers, self._tensors)):
            s, m = self._layer_structs[i], ly.mixer
            s.kind, s.has_mlp, s.heads, s.dim, s.vdim, s.ff = KIND_CODE[m.kind], int(ly.has_ff), m.heads, m.dim, m.vdim, ly.ff
            s.ff_kind = FF_CODE[ly.ff_kind]
            s.proj, s.out = _linear(t["proj_w"], t.get("proj_b")), _linear(t["out_w"], t.get("out_b"))
            s.norm1 = t["norm1"].data_ptr() if t.get("norm1") is not None else None
            s.norm1b = t["norm1b"].data_ptr() if t.get("norm1b") is not None else None
            s.act_kind, s.route_kind = ACT_CODE[ly.act], ROUTE_CODE[ly.route]
            for q in ("hc1", "hc2"):                              # read / write / mix weights of the residual streams (fp32)
                for part in ("in", "out", "mix"):
                    v = t.get(f"{q}_{part}")
                    setattr(s, f"{q}_{part}", v.data_ptr() if v is not None else None)
            if c.canon_taps > 0:
                s.canon1, s.canon_state1 = t["canon1"].data_ptr(), self.kv_cache.conv[t["conv_index"]].data_ptr()
            if m.kind == "attention":
                s.kv_heads, s.window, s.pool, s.rot_dims, s.scale = m.kv_heads, m.window, m.pool, m.rot_dims, m.scale
                s.pos_bias = t["pos_bias"].data_ptr() if t.get("pos_bias") is not None else None
                s.rot_freq = t["rot_freq"].data_ptr() if t["rot_freq"] is not None else None
                s.kv = self.kv_cache.struct(t["cache_index"])
            elif m.kind == "latent_attention":
                s.q_rank, s.kv_rank, s.rot_dim, s.rot_dims, s.scale = m.q_rank, m.kv_rank, m.rot_dim, m.rot_dims, m.scale
                s.window = m.window if m.window > 0 else 2 ** 30            # no window: every earlier position is seen
                s.rot_freq = t["rot_freq"].data_ptr() if t["rot_freq"] is not None else None
                s.uq, s.uk_t, s.uv = _linear(t["uq_w"]), t["uk_t"].data_ptr(), t["uv_w"].data_ptr()
                s.dq_norm, s.dkv_norm = t["dq_norm"].data_ptr(), t["dkv_norm"].data_ptr()
                s.sink = t["sink"].data_ptr() if t.get("sink") is not None else None
                s.kv = self.kv_cache.latent_struct(t["cache_index"])
            elif m.kind == "mingru":
                s.state = self.kv_cache.state[t["cache_index"]].data_ptr()
            elif m.kind == "attention_ssd":
                s.kv_heads, s.scale, s.window = m.kv_heads, m.scale, (m.window if m.window > 0 else 2 ** 30)
                s.q_norm = t["q_norm"].data_ptr() if t.get("q_norm") is not None else None
                s.k_norm = t["k_norm"].data_ptr() if t.get("k_norm") is not None else None
                if t.get("dist_bias") is not None:                 # fp32 [heads][n_dist], indexed by the clamped distance
                    s.dist_bias, s.n_dist = t["dist_bias"].data_ptr(), t["dist_bias"].shape[1]
                s.temp_coef, s.temp_every = float(m.temp_coef), int(m.temp_every)
                s.mix_scale_a, s.mix_scale_b = float(m.a_scale), float(m.b_scale)
                s.s_heads, s.s_vdim, s.s_state, s.s_groups = m.s_heads, m.s_vdim, m.s_state, m.s_groups
                s.s_norm_groups, s.s_taps = m.s_norm_groups, m.s_taps
                s.s_conv, s.s_norm = t["s_conv"].data_ptr(), t["s_norm"].data_ptr()
                s.s_conv_b = t["s_conv_b"].data_ptr() if t.get("s_conv_b") is not None else None
                s.s_dt_bias, s.s_a_log, s.s_d = t["s_dt_bias"].data_ptr(), t["s_a_log"].data_ptr(), t["s_d"].data_ptr()
                s.s_conv_state = self.kv_cache.mixer_conv[t["mconv_index"]].data_ptr()
                s.kv = self.kv_cache.struct(t["cache_index"])
                s.state = self.kv_cache.state[t["state_index"]].data_ptr()
            elif m.kind == "retention":
                s.rot_dims, s.rot_layout, s.qscale = m.rot_dims, ROT_LAYOUT_CODE[m.rot_layout], float(m.dim) ** -0.5
                s.rot_freq = t["rot_freq"].data_ptr() if t["rot_freq"] is not None else None
                s.decay = t["decay"].data_ptr()
                s.state = self.kv_cache.state[t["cache_index"]].data_ptr()
            elif m.kind == "attention_mlstm":
                s.kv_heads, s.scale, s.softcap = m.kv_heads, float(m.scale), float(m.softcap)
                s.window = m.window if m.window > 0 else 2 ** 30
                s.rot_dims, s.rot_layout = m.rot_dims, ROT_LAYOUT_CODE[m.rot_layout]
                s.rot_freq = t["rot_freq"].data_ptr() if t["rot_freq"] is not None else None
                s.q_norm = t["q_norm"].data_ptr() if t.get("q_norm") is not None else None
                s.k_norm = t["k_norm"].data_ptr() if t.get("k_norm") is not None else None
                s.c_taps = m.taps
                s.c_conv = t["c_conv"].data_ptr() if t.get("c_conv") is not None else None
                s.c_conv_state = self.kv_cache.mixer_conv[t["mconv_index"]].data_ptr()
                s.mix_scale_a, s.mix_scale_b, s.gate_cap = float(m.a_scale), float(m.b_scale), float(m.gate_cap)
                s.m_heads, s.m_dim, s.m_vdim, s.m_pad = m.m_heads, m.m_dim, m.m_vdim, m.m_pad
                s.m_norm = t["m_norm"].data_ptr() if t.get("m_norm") is not None else None
                s.kv = self.kv_cache.struct(t["cache_index"])
                s.state = self.kv_cache.state[t["state_index"]].data_ptr()
                s.m_max = self.kv_cache.state[t["state_index"] + 1].data_ptr()
            else:
                s.rank, s.tau, s.qscale = m.rank, m.tau, float(m.dim) ** -0.5
                s.a2, s.head_norm = _linear(t["a2_w"], t["a2_b"]), t["head_norm"].data_ptr()
                s.state = self.kv_cache.state[t["cache_index"]].data_ptr()
            s.add_embed = int(ly.add_embed)
            s.act_limit, s.shared_limit, s.act_alpha = float(ly.act_limit), float(ly.shared_limit), float(ly.act_alpha)
            if ly.has_ff:
                s.norm2 = t["norm2"].data_ptr() if t.get("norm2") is not None else None
                s.norm2b = t["norm2b"].data_ptr() if t.get("norm2b") is not None else None
                if c.canon_taps > 0:
                    s.canon2, s.canon_state2 = t["canon2"].data_ptr(), self.kv_cache.conv[t["conv_index"] + 1].data_ptr()
                if ly.ff_kind == "moe":
                    s.experts, s.top, s.expert_ff, s.shared_ff = ly.experts, ly.top, ly.expert_ff, ly.shared_ff
                    s.router, s.e_gu, s.e_down = _linear(t["router_w"], t.get("router_b")), t["e_gu"].data_ptr(), t["e_down"].data_ptr()
                    s.shared_gate = int(ly.shared_gate)
                    s.correction = t["correction"].data_ptr() if t.get("correction") is not None else None
                    if ly.shared_ff:
                        s.s_gu, s.s_down = _linear(t["s_gu_w"]), _linear(t["s_down_w"])
                else:
                    s.gu, s.down = _linear(t["gu_w"]), _linear(t["down_w"])      # polynorm: gu is the up-projection alone
                    if ly.ff_kind == "polynorm":
                        s.act = t["act"].data_ptr()
        mdl = self._m = UmbSeqModel()
        mdl.dtype, mdl.L, mdl.W, mdl.V, mdl.groups, mdl.eps = _lib.seq_dtype_code(dt), L, c.width, c.vocab_size, c.norm_groups, c.norm_eps
        mdl.embed_scale, mdl.canon_taps = float(c.embed_scale), int(c.canon_taps)
        mdl.streams, mdl.resid_mult, mdl.norm_offset = int(c.streams), float(c.resid_mult), float(c.norm_offset)
        mdl.block, mdl.logit_scale = BLOCK_CODE[c.block], float(c.logit_scale)
        mdl.embed, mdl.final_norm, mdl.head = self._top["embed"].data_ptr(), self._top["final_norm"].data_ptr(), _linear(self._top["head"])
        mdl.layers = C.cast(self._layer_structs, C.POINTER(UmbSeqLayer))
        self.reserve(self.max_step_tokens or 256)
        torch.cuda.synchronize()

    # ------------------------------------------------------------------ workspace
    def reserve(self, tokens: int, logit_rows: int | None = None):
        """Size the activation workspace for steps of up to `tokens` rows, `logit_rows` of which may ask for logits."""
        logit_rows = logit_rows or tokens
        if tokens <= self.ws_tokens and logit_rows <= self.logit_rows:
            return
        T, R = max(tokens, self.ws_tokens), max(logit_rows, self.logit_rows)
        self._graphs = {}                               # captured steps hold the old workspace's addresses
        c, dev, dt = self.config, self.device, self.dtype
        # widths of the shared scratch buffers: the largest any layer asks of each
        need = dict(proj=1, aux=1, o=1, mix=1, act=1)

        def ask(**kw):
            for k, v in kw.items():
                need[k] = max(need[k], int(v))
        top = eff = 0
        for ly, t in zip(c.layers, self._tensors):
            m = ly.mixer
            ask(proj=t["proj_w"].shape[0])
            if m.kind == "latent_attention":
                # act: query latent, then the attended latents; o: queries; mix: unrotated queries, then the gated heads;
                # aux: queries carried into the latent space
                ask(act=max(m.q_rank, m.heads * m.kv_rank), o=m.heads * (m.dim + m.rot_dim), mix=m.heads * max(m.dim, m.vdim),
                    aux=m.heads * (m.kv_rank + m.rot_dim))
            elif m.kind == "mingru":
                ask(mix=m.dim, aux=3 * m.dim + m.dim // 16 + 1)     # aux: piece summaries and start states of long stretches
            elif m.kind == "attention_ssd":
                # aux: queries | convolved [dt x | B | C | x] | decays and their logarithms | chunk states of the chunked scan
                # (one [state, vdim] matrix per head and 64 tokens, and room for a few partial chunks); o: the scan's
                # read-out; mix: [attention | state space]
                inner = m.s_heads * m.s_vdim
                chunk = m.s_heads * (m.s_state * m.s_vdim + 1)
                ask(aux=m.heads * m.dim + 2 * inner + 2 * m.s_groups * m.s_state + 2 * m.s_heads + (chunk + 63) // 64 + (8 * chunk) // T + 1,
                    o=inner, mix=m.heads * m.vdim + inner)
            elif m.kind == "retention":
                # aux: rotated [q | k] | decay rows and their logarithms | chunk states of the chunked scan
                chunk = m.heads * (m.dim * m.vdim + 1)
                ask(aux=2 * m.heads * m.dim + 2 * m.heads + (chunk + 63) // 64 + (8 * chunk + 64) // T + 1, o=m.heads * m.vdim,
                    mix=m.heads * m.vdim)
            elif m.kind == "attention_mlstm":
                # aux: queries | scaled memory queries | widened values | gates, decays, logarithms, maxima | chunk states
                # (before the memory's part begins the same room holds the convolved [q | k] row and its partial sums of few-token steps)
                chunk = m.m_heads * (m.m_dim * m.m_pad + 1)
                conv_row = (m.heads + m.kv_heads) * m.dim + 2 * (((m.heads + m.kv_heads) * m.dim + m.kv_heads * m.vdim + 255) // 256)
                ask(aux=m.heads * m.dim + max(conv_row, m.m_heads * (m.m_dim + m.m_pad + 5) + (chunk + 63) // 64 + (8 * chunk + 64) // T + 1),
                    o=m.m_heads * m.m_pad, mix=m.heads * m.vdim + m.m_heads * m.m_vdim)
            else:
                ask(aux=m.heads * m.dim, o=m.heads * m.vdim, mix=m.heads * m.vdim)
            if ly.ff_kind == "moe":
                ask(proj=ly.experts + 1, act=ly.shared_ff)
                top, eff = max(top, ly.top), max(eff, ly.expert_ff)
            elif ly.ff:
                ask(act=ly.ff, proj=ly.ff if ly.ff_kind == "polynorm" else 1)
        f32, i32 = torch.float32, torch.int32
        b = self._bufs = dict(
            x=torch.zeros(T, max(1, c.streams) * c.width, dtype=f32, device=dev), h=torch.zeros(T, c.width, dtype=dt, device=dev),
            proj=torch.zeros(T, need["proj"], dtype=f32, device=dev), aux=torch.zeros(T, need["aux"], dtype=f32, device=dev),
            o=torch.zeros(T, need["o"], dtype=f32, device=dev), mix=torch.zeros(T, need["mix"], dtype=dt, device=dev),
            act=torch.zeros(T, need["act"], dtype=dt, device=dev), y=torch.zeros(T, c.width, dtype=f32, device=dev),
            logits=torch.zeros(R, c.vocab_size, dtype=f32, device=dev))
        ws = self._ws = UmbSeqWork()
        for k in ("x", "h", "proj", "aux", "o", "mix", "act", "y", "logits"):
            setattr(ws, k, b[k].data_ptr())
        if c.block == "parallel":                       # the feed-forward's own normed input and output
            b.update(h2=torch.zeros(T, c.width, dtype=dt, device=dev), y2=torch.zeros(T, c.width, dtype=f32, device=dev))
            ws.h2, ws.y2 = b["h2"].data_ptr(), b["y2"].data_ptr()
        if top:
            pairs = T * top
            tiles = (pairs + 15) // 16 + max(ly.experts for ly in c.layers)          # the smallest tile size the forward picks
            b.update(moe_sel=torch.zeros(pairs, dtype=i32, device=dev), moe_wt=torch.zeros(pairs, dtype=f32, device=dev),
                     moe_pos=torch.zeros(pairs, dtype=i32, device=dev), moe_tiles=torch.zeros(tiles, 3, dtype=i32, device=dev),
                     moe_xs=torch.zeros(pairs, c.width, dtype=dt, device=dev), moe_act=torch.zeros(pairs, eff, dtype=dt, device=dev),
                     moe_y=torch.zeros(pairs, c.width, dtype=f32, device=dev))
            for k in ("moe_sel", "moe_wt", "moe_pos", "moe_tiles", "moe_xs", "moe_act", "moe_y"):
                setattr(ws, k, b[k].data_ptr())
            ws.moe_max_tiles = tiles
        ws.Tmax, ws.Rmax, ws.aux_floats = T, R, b["aux"].numel()
        self.ws_tokens, self.logit_rows = T, R

    @property
    def logits_buffer(self) -> torch.Tensor:
        return self._bufs["logits"]

    # ------------------------------------------------------------------ sequences
    def open(self, seq_id):
        return self.kv_cache.open(seq_id)

    def close(self, seq_id):
        self.kv_cache.close(seq_id)

    def clear(self):
        self.kv_cache.clear()

    # ------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward_batch(self, parts, want=None, trace: bool = False):
        """One step of a ragged batch.  parts: [(seq_id, token ids)], each the NEXT tokens of an open sequence; want: per
        part the indices (into that part) whose logits are asked for (default: the last one).  Returns the fp32 logits
        [rows wanted, V] (a view of the workspace, valid until the next step) in the order of parts and of want; with
        trace also the residual stream after every layer [L, T, W]."""
        cache, dev = self.kv_cache, self.device
        toks, pos, slot, seq_slot, row0, pos0, lens, rows = [], [], [], [], [], [], [], []
        for i, (sid, ids) in enumerate(parts):
            ids = [int(v) for v in (ids.tolist() if isinstance(ids, torch.Tensor) else ids)]
            n = len(ids)
            if n == 0:
                raise ValueError("a part of a step needs at least one token")
            if cache.length(sid) + n > self.max_length:
                raise RuntimeError(f"sequence {sid!r} would exceed max_length {self.max_length}")
            p0, sl = cache.extend(sid, n), cache.slot(sid)
            seq_slot.append(sl), row0.append(len(toks)), pos0.append(p0), lens.append(n)
            w = [n - 1] if want is None else list(want[i])
            rows.extend(len(toks) + int(k) for k in w)
            toks.extend(ids), pos.extend(range(p0, p0 + n)), slot.extend([sl] * n)
        T, B, R = len(toks), len(parts), len(rows)
        self.reserve(T, max(R, 1))
        host = torch.tensor(toks + pos + slot + seq_slot + row0 + pos0 + lens + rows, dtype=torch.int32)
        graphed = self.use_graph and not trace and T == B and str(dev).startswith("cuda")     # a pure decode step
        key = (T, R)
        if graphed:
            entry = self._graphs.get(key)
            if entry is None:
                entry = self._graphs[key] = {"meta": torch.zeros(host.numel(), dtype=torch.int32, device=dev), "graph": None, "runs": 0}
            meta = entry["meta"]
            meta.copy_(host)
        else:
            meta = host.to(dev)
        o = [0, T, 2 * T, 3 * T, 3 * T + B, 3 * T + 2 * B, 3 * T + 3 * B, 3 * T + 4 * B]
        p = meta.data_ptr()
        s = UmbSeqStep()
        s.T, s.B, s.R, s.max_len = T, B, R, max(lens)
        s.tokens, s.pos, s.slot, s.seq_slot, s.seq_row0, s.seq_pos0, s.seq_len, s.logit_rows = (p + 4 * v for v in o)
        tr = torch.empty(len(self.config.layers), T, self.config.width, dtype=torch.float32, device=dev) if trace else None
        s.trace = tr.data_ptr() if trace else None
        self._keep = meta

        def launch():
            rc = _lib.load_seq().umb_seq_forward(C.byref(self._m), C.byref(self._ws), C.byref(s), _lib.stream_ptr())
            if rc != 0:
                raise _lib.UmbError(f"libumbrella_seq umb_seq_forward failed with code {rc}")
        if graphed and entry["graph"] is not None:
            entry["graph"].replay()
        elif graphed and entry["runs"] >= 1:
            # the second step of this shape: everything it launches has run once (function attributes are set), so the
            # step can be captured -- capturing executes nothing -- and replayed from now on
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                launch()
            entry["graph"] = g
            g.replay()
        else:
            launch()
            if graphed:
                entry["runs"] += 1
        logits = self._bufs["logits"][:R]
        return (logits, tr) if trace else logits

    # ---- the reference's single-sequence face (umbrella/models/base.py:4-32): tokens continue ONE sequence
    _SOLO = "__solo__"

    @torch.inference_mode()
    def inference(self, input_ids, position_ids=None, attention_mask=None, storage_ids=None):
        """input_ids [1, T] continue the model's own single sequence (positions must follow on from what it holds; the
        mask and the storage ids of the tree runtime have no meaning here); returns fp32 logits [1, T, V]."""
        ids = input_ids.reshape(-1).tolist()
        if self._SOLO not in self.kv_cache.seqs:
            self.kv_cache.open(self._SOLO)
        if position_ids is not None:
            assert int(position_ids.reshape(-1)[0]) == self.kv_cache.length(self._SOLO), "positions must continue the sequence"
        return self.forward_batch([(self._SOLO, ids)], want=[list(range(len(ids)))]).clone()[None]

    def graph_inference(self, input_ids, storage_ids=None, position_ids=None, attention_mask=None):
        return self.inference(input_ids, position_ids, attention_mask, storage_ids)

    def weight_bytes(self) -> int:
        n = sum(v.numel() * v.element_size() for ly, t in zip(self.config.layers, self._tensors) if ly.weights_of is None
                for v in t.values() if isinstance(v, torch.Tensor))
        return n + self._top["head"].numel() * self._top["head"].element_size()
