"""Plain, slow torch-CPU statement of the Tomopel design (test infrastructure only; shares no code with umbrella_amd/).

One function per mechanism, whole sequences at a time, float64 unless the caller passes other tensors.  Notation: n tokens,
X the sublayer's input [n, width]; linear weights are [out, in] and applied as X @ W.T.  ``forward`` strings the mechanisms
together from a configuration dictionary (the keys of config.json) and a name -> tensor dictionary (the checkpoint's names).
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def unit_rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def offset_rms_norm(x, w, eps):
    """weight stored around zero: unit_rms(x) * (1 + w)"""
    return unit_rms(x, eps) * (1.0 + w)


# ------------------------------------------------------------------ residual streams
def streams_read(xs, w_in):
    """xs [S, n, W] -> what the sublayer's norm sees: sum_s in[s] x_s"""
    return torch.einsum("s,snw->nw", w_in, xs)


def streams_write(xs, y, w_mix, w_out, m):
    """all streams at once from the old ones: x_t <- sum_s mix[s, t] x_s + m out[t] y"""
    return torch.einsum("st,snw->tnw", w_mix, xs) + m * w_out[:, None, None] * y[None]


# ------------------------------------------------------------------ minimal gated recurrence
def min_gru(X, wz, bz, wx, bx, wg, wo, state=None):
    """z = sigmoid(Wz h + bz); u = Wx h + bx; candidate = u + 1/2 (u >= 0) or sigmoid(u) (u < 0);
    S_t = (1 - z) S_(t-1) + z candidate, element by element; out = Wo (S_t * silu(Wg h)).  Returns (out, last state)."""
    z = torch.sigmoid(X @ wz.T + bz)
    u = X @ wx.T + bx
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = silu(X @ wg.T)
    S = torch.zeros(wz.shape[0], dtype=X.dtype) if state is None else state.clone()
    outs = []
    for t in range(X.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        outs.append(S * g[t])
    return torch.stack(outs) @ wo.T, S


# ------------------------------------------------------------------ attention with a bucketed distance bias
def distance_bucket(n: int, rows: int, far: float) -> int:
    """exact below rows // 2, then logarithmic steps up to distance `far`, the last row for everything beyond"""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def biased_attention(X, wq, wk, wv, wg, wo, q_norm, k_norm, rel, *, H, G, D, E, scale, far, temp_coef, temp_every, eps,
                     pos0: int = 0, past=None):
    """Causal softmax attention, grouped query heads, unit-RMS q / k times a weight shared by the heads, a query
    temperature that grows with the position, weightless unit-RMS values, a learned bias per (distance bucket, head) added
    to the scaled scores, one sigmoid output gate per head.  past = (K, V) of earlier positions ([p, G, D], [p, G, E]);
    returns (out, (K, V))."""
    n = X.shape[0]
    q = unit_rms((X @ wq.T).reshape(n, H, D), eps) * q_norm
    k = unit_rms((X @ wk.T).reshape(n, G, D), eps) * k_norm
    v = unit_rms((X @ wv.T).reshape(n, G, E), eps)
    gate = torch.sigmoid(X @ wg.T)                                   # [n, H]
    if past is not None:
        k, v = torch.cat([past[0], k]), torch.cat([past[1], v])
    rows = rel.shape[0]
    out = torch.zeros(n, H, E, dtype=X.dtype)
    for t in range(n):
        i = pos0 + t
        temp = 1.0 + temp_coef * math.log(math.floor((i + 1) / temp_every) + 1)
        for h in range(H):
            g = h // (H // G)
            s = (k[:i + 1, g] @ (q[t, h] * temp)) * scale
            s = s + torch.stack([rel[distance_bucket(i - j, rows, far), h] for j in range(i + 1)])
            p = torch.softmax(s, 0)
            out[t, h] = (p[:, None] * v[:i + 1, g]).sum(0) * gate[t, h]
    return out.reshape(n, H * E) @ wo.T, (k, v)


# ------------------------------------------------------------------ selective state space (scalar decay per head)
def causal_conv_silu(U, w, b, history=None):
    """U [n, C]; w [C, taps] (last column: the current token); zeros before the start, or `history` [taps - 1, C]"""
    taps = w.shape[1]
    hist = torch.zeros(taps - 1, U.shape[1], dtype=U.dtype) if history is None else history
    full = torch.cat([hist, U])
    out = torch.stack([(full[t:t + taps].T * w).sum(-1) + b for t in range(U.shape[0])])
    return silu(out), full[full.shape[0] - (taps - 1):]


def ssd(X, w_in, conv_w, conv_b, dt_bias, a_log, d_skip, norm_w, wo, *, heads, vdim, state, groups, norm_groups, eps,
        past=None):
    """in-projection laid out [z | x | B | C | dt]; x, B, C through a causal convolution and silu; dt = softplus(dt + bias);
    per head S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T, y_t = S_t^T C_t + D x_t; y * silu(z), unit RMS in
    norm_groups parts, times a weight, output projection.  past = (S [heads, N, vdim], conv history); returns (out, past)."""
    n, inner, N = X.shape[0], heads * vdim, state
    p = X @ w_in.T
    z, xbc, dt = p[:, :inner], p[:, inner:2 * inner + 2 * groups * N], p[:, 2 * inner + 2 * groups * N:]
    xbc, hist = causal_conv_silu(xbc, conv_w, conv_b, None if past is None else past[1])
    x = xbc[:, :inner].reshape(n, heads, vdim)
    Bm = xbc[:, inner:inner + groups * N].reshape(n, groups, N)
    Cm = xbc[:, inner + groups * N:].reshape(n, groups, N)
    dt = softplus(dt + dt_bias)                                       # [n, heads]
    S = torch.zeros(heads, N, vdim, dtype=X.dtype) if past is None else past[0].clone()
    y = torch.zeros(n, heads, vdim, dtype=X.dtype)
    for t in range(n):
        for h in range(heads):
            g = h // (heads // groups)
            S[h] = torch.exp(-torch.exp(a_log[h]) * dt[t, h]) * S[h] + dt[t, h] * torch.outer(Bm[t, g], x[t, h])
            y[t, h] = S[h].T @ Cm[t, g] + d_skip[h] * x[t, h]
    y = y.reshape(n, inner) * silu(z)
    y = unit_rms(y.reshape(n, norm_groups, inner // norm_groups), eps).reshape(n, inner) * norm_w
    return y @ wo.T, (S, hist)


# ------------------------------------------------------------------ feed-forwards
def gated_ff(X, w_gate, w_up, w_down):
    return (silu(X @ w_gate.T) * (X @ w_up.T)) @ w_down.T


def relu2_ff(X, w_up, w_down):
    return torch.relu(X @ w_up.T).pow(2) @ w_down.T


def routed_ff(X, w_router, correction, experts, top: int, shared=None, margins=None):
    """softmax scores over all experts; the `top` largest of score + correction are chosen; weights = the chosen scores
    (without the correction) over their sum; experts = [(w_up, w_down)], each W_down relu(W_up h)^2.  margins (a list)
    collects, per token, how far the last chosen expert's choice score stands above the first one left out."""
    s = torch.softmax(X @ w_router.T, -1)
    out = torch.zeros(X.shape[0], experts[0][1].shape[0], dtype=X.dtype)
    for t in range(X.shape[0]):
        ranked = sorted(range(len(experts)), key=lambda e: (-float(s[t, e] + correction[e]), e))
        order = ranked[:top]
        if margins is not None and top < len(experts):
            margins.append(float(s[t, ranked[top - 1]] + correction[ranked[top - 1]] - s[t, ranked[top]] - correction[ranked[top]]))
        tot = sum(s[t, e] for e in order) + 1e-20
        for e in order:
            out[t] += (s[t, e] / tot) * relu2_ff(X[t:t + 1], *experts[e])[0]
    if shared is not None:
        out = out + relu2_ff(X, *shared)
    return out


# ------------------------------------------------------------------ the whole model
class State:
    """what a sequence carries from one call of ``forward`` to the next"""

    def __init__(self):
        self.pos, self.layers = 0, {}


def forward(cfg: dict, sd: dict, tokens, state: State | None = None, dtype=F, per_layer: bool = False, margins=None):
    """tokens continue the sequence that `state` describes (None: a new one).  Returns logits [n, vocab] (and, with
    per_layer, the sum of the residual streams after every layer [L, n, W])."""
    w = {k: v.to(dtype) for k, v in sd.items()}
    st = state if state is not None else State()
    eps, m, S = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0)), int(cfg.get("streams", 1))
    x = w["embed"][torch.as_tensor(tokens)] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    xs = x[None].repeat(S, 1, 1)
    trace = []

    def sublayer(xs, p, q, fn):
        hc = f"{p}hc{q}."
        if hc + "in" not in w:                                        # no stream weights: the plain residual x + m f(norm(x))
            return xs + m * fn(offset_rms_norm(xs.sum(0), w[f"{p}norm{q}"], eps))[None]
        h = offset_rms_norm(streams_read(xs, w[hc + "in"]), w[f"{p}norm{q}"], eps)
        return streams_write(xs, fn(h), w[hc + "mix"], w[hc + "out"], m)

    for i, ly in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", ly["mixer"]

        def mixer(h):
            if ly["type"] == "mingru":
                out, st.layers[i] = min_gru(h, w[p + "mix.z"], w[p + "mix.z.b"], w[p + "mix.x"], w[p + "mix.x.b"], w[p + "mix.g"],
                                            w[p + "mix.o"], st.layers.get(i))
                return out
            a, b, past = mx["left"], mx["right"], st.layers.get(i, (None, None))
            pl, pr = p + "mix.left.", p + "mix.right."
            qt = a.get("q_temp") or {"coef": 0.0, "every": 1}
            left, kv = biased_attention(h, w[pl + "q"], w[pl + "k"], w[pl + "v"], w[pl + "g"], w[pl + "o"], w[pl + "q.norm"],
                                        w[pl + "k.norm"], w[pl + "rel"], H=a["heads"], G=a.get("kv_heads", a["heads"]), D=a["dim"],
                                        E=a.get("vdim", a["dim"]), scale=a["scale"], far=a["bias_max"], temp_coef=qt["coef"],
                                        temp_every=qt["every"], eps=eps, pos0=st.pos, past=past[0])
            right, ss = ssd(h, w[pr + "in"], w[pr + "conv"], w[pr + "conv.b"], w[pr + "dt_bias"], w[pr + "A_log"], w[pr + "D"],
                            w[pr + "norm"], w[pr + "o"], heads=b["heads"], vdim=b["vdim"], state=b["state"],
                            groups=b.get("groups", 1), norm_groups=b.get("norm_groups", 1), eps=eps, past=past[1])
            st.layers[i] = (kv, ss)
            return mx.get("left_scale", 1.0) * left + mx.get("right_scale", 1.0) * right

        xs = sublayer(xs, p, 1, mixer)
        f = ly.get("mlp")
        if f is not None:
            if f["kind"] == "dense":
                xs = sublayer(xs, p, 2, lambda h: gated_ff(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"]))
            else:
                ex = [(w[p + f"mlp.e{e}.up"], w[p + f"mlp.e{e}.down"]) for e in range(f["router"]["experts"])]
                sh = (w[p + "mlp.shared.up"], w[p + "mlp.shared.down"]) if f.get("shared") else None
                corr = w.get(p + "mlp.correction", torch.zeros(len(ex), dtype=dtype))
                xs = sublayer(xs, p, 2, lambda h: routed_ff(h, w[p + "mlp.router"], corr, ex, f["router"]["top"], sh, margins))
        trace.append(xs.sum(0))
    st.pos += len(tokens)
    logits = offset_rms_norm(xs.sum(0), w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(trace)) if per_layer else logits
