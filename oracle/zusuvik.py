"""Plain, slow torch-CPU statement of the Zusuvik design (test infrastructure only; shares no code with umbrella_amd/).

One function per mechanism, float64 unless the caller passes other tensors.  Notation: n tokens, X a sublayer's input
[n, width]; linear weights are [out, in] and applied as X @ W.T.  Every mixer takes the state an earlier stretch of the same
sequence left (``None``: a sequence that starts) and returns the state it leaves, so a prompt can be fed in portions.
``forward`` strings the mechanisms together from a configuration dictionary (the keys of config.json) and a name -> tensor
dictionary (the checkpoint's names).
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def one_plus_norm(x, w, eps):
    """RMS norm whose weight is stored around zero"""
    return unit_rms(x, eps) * (1.0 + w)


# ------------------------------------------------------------------ rotary positions
def rotary_frequencies(rot: dict) -> torch.Tensor:
    """f_i = base^(-2 i / dims), i < dims / 2; with ``scaling`` the long wavelengths are slowed down by ``factor``, the
    short ones kept, and those in between blended"""
    dims = int(rot["dims"])
    i = torch.arange(dims // 2, dtype=F)
    f = float(rot["base"]) ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f.tolist():
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = torch.tensor(out, dtype=F)
    return f


def rotary(x, pos, freqs, dims: int, layout: str):
    """x [n, heads, d]; the first ``dims`` features of every head turn by pos * f_i; 'half' pairs feature i with i + dims / 2,
    'interleaved' pairs 2 i with 2 i + 1; the other features pass"""
    out = x.clone()
    half = dims // 2
    ang = pos.to(x.dtype)[:, None] * freqs.to(x.dtype)[None, :]          # [n, dims / 2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    if layout == "half":
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------ retention
def retention(X, pos, m: dict, w: dict, eps: float, state=None):
    """linear attention with one fixed decay per head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, no softmax and no
    denominator; rotary (half layout) on q and k, k scaled by dim^-1/2 after it; every head's o over its root mean square, the
    heads side by side times silu(W_g h), then W_o.  w: q, k, v, g, o.  Returns (out, state [heads, dim, vdim])."""
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    n = X.shape[0]
    q, k = (X @ w["q"].T).view(n, H, D), (X @ w["k"].T).view(n, H, D)
    if m.get("rot") and int(m["rot"]["dims"]) > 0:
        fr = rotary_frequencies(m["rot"])
        q, k = (rotary(z, pos, fr, int(m["rot"]["dims"]), "half") for z in (q, k))
    k = k * D ** -0.5
    v = (X @ w["v"].T).view(n, H, Dv)
    decay = torch.tensor([float(d) for d in m["decay"]], dtype=X.dtype)
    S = torch.zeros(H, D, Dv, dtype=X.dtype) if state is None else state.clone()
    o = torch.zeros(n, H, Dv, dtype=X.dtype)
    for t in range(n):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hdv,hd->hv", S, q[t])
    y = unit_rms(o, eps).reshape(n, H * Dv) * silu(X @ w["g"].T)
    return y @ w["o"].T, S


# ------------------------------------------------------------------ short causal convolution over time
def causal_conv(U, taps_w, history=None):
    """U [n, channels]; taps_w [channels, taps]; y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the sequence's start.
    history: the last taps - 1 inputs of earlier stretches [taps - 1, channels].  Returns (y, new history)."""
    taps = taps_w.shape[1]
    n, C = U.shape
    hist = torch.zeros(taps - 1, C, dtype=U.dtype) if history is None else history
    ext = torch.cat([hist, U], dim=0)                                    # position t of U is row t + taps - 1
    y = torch.zeros_like(U)
    for j in range(taps):
        y = y + taps_w[:, j][None, :] * ext[j:j + n]
    return y, ext[ext.shape[0] - (taps - 1):].clone()


# ------------------------------------------------------------------ softmax attention with a capped score
def capped_attention(q, k, v, q_pos, scale: float, softcap: float):
    """q [n, H, D] at positions q_pos; k [m, G, D], v [m, G, E] of positions 0 .. m - 1; query head h reads key / value head
    h // (H / G); score = softcap tanh(q . k scale / softcap); position i sees every j <= i.  Returns [n, H, E]."""
    n, H, _ = q.shape
    m_, G, E = v.shape
    out = torch.zeros(n, H, E, dtype=q.dtype)
    kpos = torch.arange(m_)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(kpos[None, :] > q_pos[:, None], -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def conv_attention(X, pos, m: dict, w: dict, eps: float, state=None):
    """grouped-query softmax attention whose q, k, v (projected with biases) first pass a short causal convolution per channel,
    then q and k an RMS norm over the WHOLE projection (plain weights), then interleaved rotary with scaled frequencies.
    state: {"hist": [taps - 1, channels of q | k | v], "k": [m, G, D], "v": [m, G, E]}."""
    H, G, D, E = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    n = X.shape[0]
    raw = torch.cat([X @ w["q"].T + w["q.b"], X @ w["k"].T + w["k.b"], X @ w["v"].T + w["v.b"]], dim=1)
    taps_w = torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]], dim=0)
    st = state or {}
    u, hist = causal_conv(raw, taps_w, st.get("hist"))
    q, k, v = u[:, :H * D], u[:, H * D:H * D + G * D], u[:, H * D + G * D:]
    q = unit_rms(q, eps) * w["q.norm"]
    k = unit_rms(k, eps) * w["k.norm"]
    fr = rotary_frequencies(m["rot"])
    q = rotary(q.reshape(n, H, D), pos, fr, int(m["rot"]["dims"]), "interleaved")
    k = rotary(k.reshape(n, G, D), pos, fr, int(m["rot"]["dims"]), "interleaved")
    v = v.reshape(n, G, E)
    if st.get("k") is not None:
        k, v = torch.cat([st["k"], k]), torch.cat([st["v"], v])
    o = capped_attention(q, k, v, pos, float(m["scale"]), float(m["softcap"]))
    return o.reshape(n, H * E) @ w["o"].T + w["o.b"], {"hist": hist, "k": k, "v": v}


# ------------------------------------------------------------------ matrix memory with exponential gates
def matrix_memory(X, m: dict, w: dict, eps: float, state=None):
    """per head: log input gate i = cap tanh(z_i / cap), log forget gate f = logsigmoid(cap tanh(z_f / cap)); a running
    maximum m (starts at 0) keeps the exponentials in range:
        m_t = max(f + m_(t-1), i);  S_t = e^(f + m_(t-1) - m_t) S_(t-1) + e^(i - m_t) k v^T;  n_t the same with k alone;
        o_t = S_t^T q / (max(|n_t . q|, e^(-m_t)) + 1e-6),  q scaled by dim^-1/2.
    Every head's o over its root mean square, times the norm weight (all heads), times sigmoid(W_g h), then W_o.
    state: (S [H, D, Dv], n [H, D], m [H])."""
    H, D, Dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    n_tok = X.shape[0]
    q = (X @ w["q"].T).view(n_tok, H, D) * D ** -0.5
    k = (X @ w["k"].T).view(n_tok, H, D)
    v = (X @ w["v"].T).view(n_tok, H, Dv)
    gi = cap * torch.tanh((X @ w["i"].T + w["i.b"]) / cap)
    gf = torch.nn.functional.logsigmoid(cap * torch.tanh((X @ w["f"].T + w["f.b"]) / cap))
    if state is None:
        S, nn, mm = torch.zeros(H, D, Dv, dtype=X.dtype), torch.zeros(H, D, dtype=X.dtype), torch.zeros(H, dtype=X.dtype)
    else:
        S, nn, mm = (s.clone() for s in state)
    o = torch.zeros(n_tok, H, Dv, dtype=X.dtype)
    for t in range(n_tok):
        m_new = torch.maximum(gf[t] + mm, gi[t])
        a, b = torch.exp(gf[t] + mm - m_new), torch.exp(gi[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        nn = a[:, None] * nn + b[:, None] * k[t]
        mm = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((nn * q[t]).sum(-1).abs(), torch.exp(-mm)) + 1e-6
        o[t] = num / den[:, None]
    y = unit_rms(o, eps).reshape(n_tok, H * Dv) * w["norm"] * torch.sigmoid(X @ w["g"].T)
    return y @ w["o"].T, (S, nn, mm)


# ------------------------------------------------------------------ experts
def capped_glu_expert(X, w_gate, w_up, w_down, limit: float):
    """g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))"""
    g = torch.clamp(X @ w_gate.T, max=limit)
    u = torch.clamp(X @ w_up.T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route_top_logits(z, top: int):
    """the ``top`` largest logits of every row (ties: the lower index) and the softmax over just those"""
    order = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.softmax(torch.gather(z, 1, order), dim=-1)


def expert_mixture(X, mlp: dict, w: dict, margins=None):
    """routed experts (weights = softmax over the chosen logits, applied to the experts' outputs) plus, where the
    configuration has one, a shared expert times sigmoid(W_sg h), one number per token.  margins (a list): gets, per token, how
    far the last chosen logit stands above the first one not chosen."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    limit = float(mlp["expert"]["limit"])
    z = X @ w["router"].T + w["router.b"]
    sel, wt = route_top_logits(z, top)
    if margins is not None and top < E:
        srt = torch.sort(z, dim=-1, descending=True).values
        margins.extend((srt[:, top - 1] - srt[:, top]).tolist())
    y = torch.zeros(X.shape[0], w["e0.down"].shape[0], dtype=X.dtype)
    for e in range(E):
        for c in range(top):
            rows = (sel[:, c] == e).nonzero().flatten()
            if rows.numel():
                y[rows] += wt[rows, c][:, None] * capped_glu_expert(X[rows], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], limit)
    if mlp.get("shared"):
        ys = capped_glu_expert(X, w["shared.gate"], w["shared.up"], w["shared.down"], float(mlp["shared"]["limit"]))
        y = y + torch.sigmoid(X @ w["shared.sg"].T) * ys
    return y


# ------------------------------------------------------------------ the model
def layer_runs(cfg: dict):
    """[(layer index, first of a repeated pass)] in the order the layers run: layers start .. stop - 1 run ``times`` times in a
    row, the rest once"""
    L = len(cfg["layers"])
    lp = cfg.get("loop") or {}
    start, stop, times = int(lp.get("start", 0)), int(lp.get("stop", 0)), int(lp.get("times", 1))
    if stop <= start or times <= 1:
        return [(i, False) for i in range(L)]
    runs = [(i, False) for i in range(start)]
    for p in range(times):
        runs += [(i, p > 0 and i == start) for i in range(start, stop)]
    return runs + [(i, False) for i in range(stop, L)]


def _sub(sd: dict, prefix: str, dtype) -> dict:
    return {k[len(prefix):]: v.to(dtype) for k, v in sd.items() if k.startswith(prefix)}


def forward(cfg: dict, sd: dict, tokens, state=None, dtype=F, margins=None):
    """tokens: the next ids of ONE sequence; state: what ``forward`` returned for the stretch before (None: the sequence
    starts).  Returns (logits [n, vocab], residual stream after every layer run [runs, n, width], state)."""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    n = ids.numel()
    state = state or {"len": 0, "runs": {}}
    pos = torch.arange(state["len"], state["len"] + n)
    emb = sd["embed"].to(dtype)
    x0 = emb[ids]
    x = x0.clone()
    trace, new_runs = [], {}
    for r, (i, again) in enumerate(layer_runs(cfg)):
        ly = cfg["layers"][i]
        p = f"l{i}."
        if again:
            x = x + x0
        h = one_plus_norm(x, sd[p + "norm1"].to(dtype), eps)
        st = state["runs"].get(r)
        if ly["type"] == "retention":
            y, ns = retention(h, pos, ly["mixer"], _sub(sd, p + "mix.", dtype), eps, st)
        elif ly["type"] == "parallel":
            st = st or (None, None)
            ya, sa = conv_attention(h, pos, ly["mixer"]["left"], _sub(sd, p + "mix.left.", dtype), eps, st[0])
            yb, sb = matrix_memory(h, ly["mixer"]["right"], _sub(sd, p + "mix.right.", dtype), eps, st[1])
            y, ns = float(ly["mixer"]["left_scale"]) * ya + float(ly["mixer"]["right_scale"]) * yb, (sa, sb)
        else:
            raise ValueError(ly["type"])
        new_runs[r] = ns
        if ly.get("mlp"):
            h2 = one_plus_norm(x, sd[p + "norm2"].to(dtype), eps)
            y = y + expert_mixture(h2, ly["mlp"], _sub(sd, p + "mlp.", dtype), margins)
        x = x + y
        trace.append(x.clone())
    logits = one_plus_norm(x, sd["final.norm"].to(dtype), eps) @ emb.T * float(cfg["logit_scale"])
    return logits, torch.stack(trace), {"len": state["len"] + n, "runs": new_runs}
