"""The Zusuvik design on the HIP path against the plain oracle (oracle/zusuvik.py): its mechanisms alone through their own
entry points of libumbrella_seq.so (the parallel-block seam, rotary layouts, retention on the linear scans, the convolved
attention front end with capped scores, the matrix memory with its running maximum, routing on the logits with the capped gated
experts and the gated shared expert), then whole models through the runtime, the cache manager, the batch engine and the trace
replay command.

fp32 runs are the sharp ones (every comparison to ~1e-5: one key too many, a lost state or a tap from the wrong position is a
thousand times that); bf16 runs use inputs built so that a fault still shows."""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
F32_TOL = 2e-5
BF16_TOL = 4e-2
D64 = torch.float64


@pytest.fixture(scope="module")
def lib():
    import __graft_entry__ as ge
    from umbrella_amd import _lib
    if not os.path.exists(_lib.SEQ_LIB_PATH):
        ge.build_seq()
    return _lib.load_seq()


def dev(t, dtype=None):
    return t.to(device="cuda:0", dtype=dtype).contiguous()


def i32(v):
    return torch.tensor(v, dtype=torch.int32, device="cuda:0")


def zeros(*shape, dtype=torch.float32):
    return torch.zeros(*shape, dtype=dtype, device="cuda:0")


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30)) < tol


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def row_errs(got, want):
    """rel_err row by row"""
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rnd(shape, seed, scale=1.0):
    return scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))


def code(dtype):
    from umbrella_amd import _lib
    return _lib.seq_dtype_code(dtype)


def call(name, *a):
    from umbrella_amd import _lib
    return _lib.seq_call(name, *a)


class Steps:
    """the index arrays of a step for sequences that each bring `counts[b]` rows from position `pos0[b]` in slot `slots[b]`"""

    def __init__(self, counts, pos0, slots):
        self.pos, self.slot, self.row0 = [], [], []
        for n, p, s in zip(counts, pos0, slots):
            self.row0.append(len(self.pos))
            self.pos += list(range(p, p + n))
            self.slot += [s] * n
        self.T, self.B, self.max_len = len(self.pos), len(counts), max(counts)
        self.d = dict(pos=i32(self.pos), slot=i32(self.slot), seq_slot=i32(slots), seq_row0=i32(self.row0), seq_pos0=i32(pos0),
                      seq_len=i32(counts))


# ------------------------------------------------------------------ the seam of parallel blocks
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("W,T", [(40, 3), (300, 5), (1500, 2), (3000, 2), (5000, 1)])
def test_parallel_block_seam_and_embedding(lib, dtype, W, T):
    V, eps, off, es = 17, 1e-5, 1.0, 1.0
    emb = rnd((V, W), 1).to(dtype)
    tk = tokens(T, V, 2)
    w1, w2 = rnd((W,), 3, 0.2).to(dtype), rnd((W,), 4, 0.2).to(dtype)
    y1, y2 = rnd((T, W), 5), rnd((T, W), 6)
    tol = 1e-6 if dtype == torch.float32 else 1e-2

    def norm(x, w):
        x = x.double()
        return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (off + w.double())
    x, h1, h2 = zeros(T, W), zeros(T, W, dtype=dtype), zeros(T, W, dtype=dtype)
    call("umb_blk_seam", x, h1, h2, None, None, dev(emb), i32(tk), 1, es, dev(w1), dev(w2), off, T, W, V, eps, code(dtype))
    x0 = emb[tk].float()
    assert torch.equal(x.cpu(), x0) and close(h1, norm(x0, w1), tol) and close(h2, norm(x0, w2), tol)
    # both outputs join together; only the first norm is wanted
    h2.zero_()
    call("umb_blk_seam", x, h1, None, dev(y1), dev(y2), None, None, 0, 0.0, dev(w1), None, off, T, W, V, eps, code(dtype))
    x1 = x0 + (y1 + y2)
    assert close(x, x1, 1e-6) and close(h1, norm(x1, w1), tol) and float(h2.abs().max()) == 0.0
    # the embedding row joins again in front of a repeated span; a layer without feed-forward brings one output
    call("umb_blk_seam", x, h1, h2, dev(y1), None, dev(emb), i32(tk), 2, es, dev(w1), dev(w2), off, T, W, V, eps, code(dtype))
    x2 = (x1 + y1) + x0
    assert close(x, x2, 1e-6) and close(h2, norm(x2, w2), tol)
    # no norm at all: the residual alone moves
    call("umb_blk_seam", x, None, None, None, dev(y2), None, None, 0, 0.0, None, None, off, T, W, V, eps, code(dtype))
    assert close(x, x2 + y2, 1e-6)


@pytest.mark.parametrize("D,dims,layout", [(8, 8, "half"), (8, 4, "half"), (7, 6, "interleaved"), (16, 16, "interleaved"), (5, 0, "half"),
                                          (64, 32, "half")])
def test_rotary_of_both_layouts_with_constants(lib, D, dims, layout):
    from oracle import zusuvik as O
    from umbrella_amd.models.config import rotary_frequencies
    T, heads, ha = 9, 5, 2
    x = rnd((T, heads * D + 3), 1)
    pos = [0, 1, 2, 700, 701, 5, 63, 64, 1023]
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    fr = rotary_frequencies(50.0, dims, sc) if dims else None
    out = zeros(T, heads * D)
    call("umb_rope_scale", out, heads * D, dev(x), heads * D + 3, i32(pos), dev(fr) if dims else None, T, heads, D, dims,
         0 if layout == "half" else 1, ha, 0.5, 3.0)
    xs = x[:, :heads * D].double().view(T, heads, D)
    want = O.rotary(xs, torch.tensor(pos), O.rotary_frequencies({"base": 50.0, "dims": dims, "scaling": sc}), dims, layout) if dims else xs.clone()
    want[:, :ha] *= 0.5
    want[:, ha:] *= 3.0
    assert close(out.view(T, heads, D), want, 3e-5)          # fp32 angles at position ~1000: a few 1e-5 of a radian


# ------------------------------------------------------------------ retention
def _scan(lib, o, state, q, ldq, k, ldk, v, ldv, alpha, la, st, H, D, P, scratch):
    """as the forward chooses: chunks for stretches of 64 tokens and more, token by token otherwise"""
    need = lib.umb_ssd_scan_chunked_floats(st.B, st.max_len, H, D, P) if st.max_len >= 64 else 0
    if need and need <= scratch.numel():
        call("umb_ssd_scan_chunked", o, state, q, ldq, k, ldk, v, ldv, la, H, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
             st.d["seq_len"], st.B, st.max_len, H, D, P, scratch, scratch.numel())
    else:
        call("umb_lin_scan", o, state, q, ldq, k, ldk, v, ldv, alpha, 1, H, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
             st.d["seq_len"], st.B, H, D, P, 1.0)


def _offset(t, n):
    """the tensor from element n on (same storage), for passing column offsets as pointers"""
    return t.view(-1)[n:]


def _run_retention(lib, m, w, X, splits, dtype, slot=1, state=None):
    from umbrella_amd.models.config import rotary_frequencies
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    dims = m.get("rot", {}).get("dims", 0)
    fr = dev(rotary_frequencies(m["rot"]["base"], dims)) if dims else None
    proj_all = (X.double() @ torch.cat([w["q"], w["k"], w["v"], w["g"]]).double().T).float()
    ld = proj_all.shape[1]
    state = zeros(3, H, D, Dv) + 7.0 if state is None else state          # a fresh sequence must not read what the slot holds
    decay = dev(torch.tensor(m["decay"], dtype=torch.float32))
    scratch = zeros(1 << 20)
    outs, at = [], 0
    for cnt in splits:
        st = Steps([cnt], [at], [slot])
        proj = dev(proj_all[at:at + cnt])
        qk, alpha, la = zeros(cnt, 2 * H * D), zeros(cnt, H), zeros(cnt, H)
        o, out = zeros(cnt, H * Dv), zeros(cnt, H * Dv + 2, dtype=dtype)
        call("umb_rope_scale", qk, 2 * H * D, proj, ld, st.d["pos"], fr, cnt, 2 * H, D, dims, 0, H, 1.0, D ** -0.5)
        call("umb_decay_fill", alpha, la, decay, cnt, H)
        _scan(lib, o, state, qk, 2 * H * D, _offset(qk, H * D), 2 * H * D, _offset(proj, 2 * H * D), ld, alpha, la, st, H, D, Dv, scratch)
        call("umb_head_gate", out, H * Dv + 2, o, Dv, -1, None, proj, ld, 2 * H * D + H * Dv, None, 0, 0, cnt, H, Dv, 1e-5, 1.0, code(dtype))
        assert float(out[:, H * Dv:].abs().max()) == 0.0
        outs.append(out[:, :H * Dv].clone())
        at += cnt
    return torch.cat(outs), state


def _retention_case(H, D, Dv, rot, seed, n, W=24):
    m = {"heads": H, "dim": D, "vdim": Dv, "decay": [1.0 - 0.3 / (h + 1) ** 2 for h in range(H)]}
    if rot:
        m["rot"] = {"base": 200.0, "dims": rot}
    w = {"q": rnd((H * D, W), seed) / W ** 0.5, "k": rnd((H * D, W), seed + 1) / W ** 0.5, "v": rnd((H * Dv, W), seed + 2) / W ** 0.5,
         "g": rnd((H * Dv, W), seed + 3) / W ** 0.5, "o": torch.eye(H * Dv)}
    return m, w, rnd((n, W), seed + 4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,Dv,rot,splits", [(3, 8, 6, 8, [19]), (2, 5, 3, 0, [1] * 12), (4, 16, 16, 8, [2, 9, 1, 1, 17, 3]),
                                               (1, 7, 9, 6, [2, 2, 2]), (2, 32, 20, 32, [40, 1, 1])])
def test_retention_prompt_portions_and_single_tokens(lib, dtype, H, D, Dv, rot, splits):
    from oracle import zusuvik as O
    m, w, X = _retention_case(H, D, Dv, rot, 1, sum(splits))
    want, S = O.retention(X.double(), torch.arange(sum(splits)), m, {k: v.double() for k, v in w.items()}, 1e-5)
    got, state = _run_retention(lib, m, w, X, splits, dtype)
    assert close(got, want, F32_TOL if dtype == torch.float32 else 1e-2)
    assert close(state[1], S, F32_TOL) and float((state[0] - 7.0).abs().max()) == 0.0


@pytest.mark.parametrize("H,D,Dv,rot,splits", [(3, 8, 6, 8, [150]), (2, 32, 20, 16, [70, 1, 1, 64, 3, 130]), (2, 130, 5, 0, [64, 65])])
def test_retention_long_stretches_in_chunks(lib, H, D, Dv, rot, splits):
    from oracle import zusuvik as O
    m, w, X = _retention_case(H, D, Dv, rot, 11, sum(splits))
    m["decay"][0] = 1.0                                   # nothing is forgotten: the first token still counts at the end
    want, S = O.retention(X.double(), torch.arange(sum(splits)), m, {k: v.double() for k, v in w.items()}, 1e-5)
    got, state = _run_retention(lib, m, w, X, splits, torch.float32)
    assert close(got, want, F32_TOL) and close(state[1], S, F32_TOL)
    again, _ = _run_retention(lib, m, w, X, [1] * 40, torch.float32, state=state)       # the slot is used again from position 0
    assert close(again, want[:40], F32_TOL)


# ------------------------------------------------------------------ convolved attention with capped scores
def _run_conv_attention(lib, m, w, X, splits, dtype, page=4, cache=None, seq="s", raw=None, split_rows=True):
    from umbrella_amd.attn.cache import PagedSeqCache
    from umbrella_amd.models.config import rotary_frequencies
    H, G, D, E, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    C = H * D + G * D + G * E
    rot = m["rot"]
    fr = dev(rotary_frequencies(rot["base"], rot["dims"], rot.get("scaling"))) if rot["dims"] else None
    if raw is None:
        raw = torch.cat([X.double() @ w["q"].double().T + w["q.b"].double(), X.double() @ w["k"].double().T + w["k.b"].double(),
                         X.double() @ w["v"].double().T + w["v.b"].double()], dim=1)
    proj_all = torch.cat([raw.float(), torch.full((raw.shape[0], 2), 9.0)], dim=1)       # columns behind the three are not touched
    ld = C + 2
    if cache is None:
        cache = PagedSeqCache([(G, D, 0, E)], [], 1024, 3, "cuda:0", dtype, page=page, mixer_convs=[(taps, C)])
        cache.mixer_conv[0].fill_(5.0)                    # a fresh sequence must not read what the ring holds
    cache.open(seq)
    kv = cache.struct(0)
    conv = dev(torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]]), dtype)
    scratch2 = zeros(64 * (C + 64))                       # with it, steps of few tokens convolve over (token, 256 channels)
    outs, at = [], 0
    for cnt in splits:
        p0 = cache.extend(seq, cnt)
        st = Steps([cnt], [p0], [cache.slot(seq)])
        proj = dev(proj_all[at:at + cnt])
        q, out = zeros(cnt, H * D), zeros(cnt, H * E + 3, dtype=dtype)
        single = int(cnt == 1)
        call("umb_cva_prep", q, kv, proj, ld, conv, cache.mixer_conv[0], dev(w["q.norm"], dtype), dev(w["k.norm"], dtype), st.d["pos"],
             st.d["slot"], fr, cnt, H, G, D, E, taps, rot["dims"], 1, single, 1e-5, scratch2 if split_rows else None,
             scratch2.numel() if split_rows else 0, code(dtype))
        if not single:
            call("umb_ssd_conv_update", cache.mixer_conv[0], proj, ld, 0, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
                 st.d["seq_len"], 1, C, taps)
        if cnt >= 16 and lib.umb_bsa_attend_tiled_ok(H, G, D, E, code(dtype)):
            call("umb_bsa_attend_tiled", out, H * E + 3, q, kv, proj, ld, -1, None, 0, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
                 st.d["seq_len"], 1, cnt, H, G, D, E, 2 ** 30, m["scale"], 0.8, m["softcap"], code(dtype))
        else:
            scratch = zeros(cnt * H * 16 * (E + 2))
            call("umb_bsa_attend", out, H * E + 3, q, kv, proj, ld, -1, None, 0, st.d["pos"], st.d["slot"], cnt, H, G, D, E, 2 ** 30,
                 m["scale"], 0.8, m["softcap"], scratch, scratch.numel(), code(dtype))
        assert float(out[:, H * E:].abs().max()) == 0.0
        outs.append(out[:, :H * E].clone())
        at += cnt
    return torch.cat(outs), cache


def _conv_attention_case(H, G, D, E, taps, dims, scaling, softcap, seed, n, W=24):
    rot = {"base": 80.0, "dims": dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": E, "conv": taps, "rot": rot, "scale": D ** -0.5, "softcap": softcap}
    C = [H * D, G * D, G * E]
    w = {"q": rnd((C[0], W), seed) / W ** 0.5, "k": rnd((C[1], W), seed + 1) / W ** 0.5, "v": rnd((C[2], W), seed + 2) / W ** 0.5,
         "q.b": rnd((C[0],), seed + 3, 0.3), "k.b": rnd((C[1],), seed + 4, 0.3), "v.b": rnd((C[2],), seed + 5, 0.3),
         "q.conv": rnd((C[0], taps), seed + 6, 0.6), "k.conv": rnd((C[1], taps), seed + 7, 0.6), "v.conv": rnd((C[2], taps), seed + 8, 0.6),
         "q.norm": 1 + rnd((C[0],), seed + 9, 0.2), "k.norm": 1 + rnd((C[1],), seed + 10, 0.2), "o": torch.eye(H * E), "o.b": torch.zeros(H * E)}
    return m, w, rnd((n, W), seed + 11)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,taps,dims,scaling,softcap,splits",
                         [(4, 2, 8, 6, 3, 4, True, 3.0, [19]), (3, 1, 7, 9, 1, 6, False, 50.0, [1] * 11), (2, 2, 16, 16, 4, 16, True, 2.0, [2, 2, 7, 1, 1, 16, 3]),
                          (8, 2, 32, 48, 2, 8, True, 4.0, [30, 1, 1, 17, 2, 70, 1]), (4, 4, 8, 16, 5, 0, False, 8.0, [3, 2, 2, 1, 1, 1, 6]),
                          (2, 1, 8, 8, 9, 4, False, 6.0, [5, 1, 1, 4, 1, 12])])
def test_convolved_attention_prompt_portions_and_single_tokens(lib, dtype, H, G, D, E, taps, dims, scaling, softcap, splits):
    from oracle import zusuvik as O
    n = sum(splits)
    m, w, X = _conv_attention_case(H, G, D, E, taps, dims, scaling, softcap, 1, n)
    wd = {k: v.to(dtype).double() for k, v in w.items()}
    want, _ = O.conv_attention(X.double(), torch.arange(n), m, wd, 1e-5)
    got, cache = _run_conv_attention(lib, m, {k: v.to(dtype).float() for k, v in w.items()}, X, splits, dtype)
    assert close(got, 0.8 * want, F32_TOL if dtype == torch.float32 else BF16_TOL)
    one, _ = _run_conv_attention(lib, m, {k: v.to(dtype).float() for k, v in w.items()}, X, splits, dtype, split_rows=False)
    assert close(one, 0.8 * want, F32_TOL if dtype == torch.float32 else BF16_TOL)       # one workgroup per token whatever the step
    # the pages and the slot go back and are used again by a sequence that starts at 0
    cache.close("s")
    again, _ = _run_conv_attention(lib, m, {k: v.to(dtype).float() for k, v in w.items()}, X[:9], [4, 1, 4], dtype, cache=cache, seq="t")
    assert close(again, 0.8 * want[:9], F32_TOL if dtype == torch.float32 else BF16_TOL)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_convolved_attention_finds_one_far_key_and_nothing_ahead(lib, dtype):
    """one key row far back points along the query's direction, all others against it (the whole-row norm keeps directions; the
    capped scores are +cap for that key and -cap for the rest), its value row carries a mark: queries at and after it read the mark, queries before it do not -- in a long
    prompt (matrix pipe in 16 bits), across page borders, and for tokens decoded one by one"""
    from oracle import zusuvik as O
    H, G, D, E, n, far = 4, 2, 16, 16, 420, 5
    m, w, _ = _conv_attention_case(H, G, D, E, 1, 0, False, 12.0, 3, n)
    for k in ("q.conv", "k.conv", "v.conv"):
        w[k] = torch.ones_like(w[k])
    w["q.norm"], w["k.norm"] = torch.ones(H * D), torch.ones(G * D)
    raw = rnd((n, H * D + G * D + G * E), 4, 0.05)
    raw[:, :H * D] += 1.0                                 # every query points along (1, 1, ..): so does key `far` alone,
    raw[:, H * D:H * D + G * D] -= 1.0                    # every other key points the opposite way
    raw[far, H * D:H * D + G * D] = 3.0
    raw[:, H * D + G * D:] = rnd((n, G * E), 5, 0.01)
    raw[far, H * D + G * D:] = 7.0
    m["scale"] = 2.0
    wd = {k: v.double() for k, v in w.items()}
    q = O.unit_rms(raw[:, :H * D].double(), 1e-5).view(n, H, D)
    k = O.unit_rms(raw[:, H * D:H * D + G * D].double(), 1e-5).view(n, G, D)
    ref = O.capped_attention(q, k, raw[:, H * D + G * D:].double().view(n, G, E), torch.arange(n), 2.0, 12.0).reshape(n, H * E)
    for splits in ([n], [380] + [1] * 40, [3, 2, 250, 165]):
        got, _ = _run_conv_attention(lib, m, wd, None, splits, dtype, raw=raw.double())
        assert close(got, 0.8 * ref, F32_TOL if dtype == torch.float32 else BF16_TOL)
        assert float(got[:far].float().abs().max()) < 0.2 and float(got[far:].float().min()) > 4.0      # 0.8 * 7, nearly all of it


# ------------------------------------------------------------------ matrix memory
def _run_memory(lib, m, w, X, splits, dtype, slot=2, state=None):
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    Pp = (Dv + 1 + 3) // 4 * 4
    X = X.double()
    proj_all = torch.cat([X @ w["q"].double().T, X @ w["k"].double().T, X @ w["v"].double().T, X @ w["g"].double().T,
                          X @ w["i"].double().T + w["i.b"].double(), X @ w["f"].double().T + w["f.b"].double()], dim=1).float()
    ld = proj_all.shape[1]
    qc, kc, vc, gc, ic, fc = 0, H * D, 2 * H * D, 2 * H * D + H * Dv, 2 * H * D + 2 * H * Dv, 2 * H * D + 2 * H * Dv + H
    if state is None:
        state = (zeros(3, H, D, Pp) + 3.0, zeros(3, H) - 2.0)                # a fresh sequence must not read what the slot holds
    S, mx = state
    scratch = zeros(1 << 20)
    outs, at = [], 0
    for cnt in splits:
        st = Steps([cnt], [at], [slot])
        proj = dev(proj_all[at:at + cnt])
        qs, vp, bw = zeros(cnt, H * D), zeros(cnt, H * Pp), zeros(cnt, H)
        alpha, la, mrun = zeros(cnt, H), zeros(cnt, H), zeros(cnt, H)
        o, out = zeros(cnt, H * Pp), zeros(cnt, H * Dv + 2, dtype=dtype)
        if cnt == 1:
            call("umb_mlstm_step", qs, vp, la, alpha, mrun, mx, proj, ld, qc, vc, ic, fc, st.d["pos"], st.d["slot"], cnt, H, D, Dv, Pp,
                 D ** -0.5, cap)
        else:
            call("umb_mlstm_mscan", la, alpha, mrun, bw, mx, proj, ld, ic, fc, cap, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
                 st.d["seq_len"], 1, H)
            call("umb_mlstm_prep", qs, vp, proj, ld, qc, vc, bw, cnt, H, D, Dv, Pp, D ** -0.5)
        _scan(lib, o, S, qs, H * D, _offset(proj, kc), ld, vp, H * Pp, alpha, la, st, H, D, Pp, scratch)
        call("umb_head_gate", out, H * Dv + 2, o, Pp, Dv, mrun, proj, ld, gc, dev(w["norm"], dtype), 1, 1, cnt, H, Dv, 1e-5, 1.2, code(dtype))
        assert float(out[:, H * Dv:].abs().max()) == 0.0
        outs.append(out[:, :H * Dv].clone())
        at += cnt
    return torch.cat(outs), (S, mx)


def _memory_case(H, D, Dv, cap, seed, n, W=24, gate_gain=2.0):
    m = {"heads": H, "dim": D, "vdim": Dv, "gate_cap": cap}
    w = {"q": rnd((H * D, W), seed) / W ** 0.5, "k": rnd((H * D, W), seed + 1) / W ** 0.5, "v": rnd((H * Dv, W), seed + 2) / W ** 0.5,
         "g": rnd((H * Dv, W), seed + 3) / W ** 0.5, "i": gate_gain * rnd((H, W), seed + 4) / W ** 0.5, "f": gate_gain * rnd((H, W), seed + 5) / W ** 0.5,
         "i.b": rnd((H,), seed + 6), "f.b": 1.0 + rnd((H,), seed + 7), "norm": 1 + rnd((H * Dv,), seed + 8, 0.2), "o": torch.eye(H * Dv)}
    return m, w, rnd((n, W), seed + 9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,Dv,cap,gain,splits", [(3, 5, 7, 6.0, 2.0, [19]), (2, 3, 3, 2.0, 8.0, [1] * 12), (6, 32, 48, 12.0, 2.0, [2, 9, 1, 1, 17, 3]),
                                                    (1, 7, 4, 1.0, 20.0, [2, 2, 2, 1]), (2, 16, 11, 30.0, 40.0, [40, 1, 1])])
def test_matrix_memory_prompt_portions_and_single_tokens(lib, dtype, H, D, Dv, cap, gain, splits):
    """gains large enough that the caps bind and the running maximum moves both ways (it starts at 0, not at the first gate)"""
    from oracle import zusuvik as O
    n = sum(splits)
    m, w, X = _memory_case(H, D, Dv, cap, 1, n, gate_gain=gain)
    want, (S, nn, mm) = O.matrix_memory(X.double(), m, {k: v.to(dtype).double() if k == "norm" else v.double() for k, v in w.items()}, 1e-5)
    got, (state, mx) = _run_memory(lib, m, w, X, splits, dtype)
    assert close(got, 1.2 * want, F32_TOL if dtype == torch.float32 else 1e-2)
    assert close(state[2][:, :, :Dv], S, F32_TOL) and close(state[2][:, :, Dv], nn, F32_TOL) and close(mx[2], mm, 1e-6)
    assert float((state[0] - 3.0).abs().max()) == 0.0 and float((mx[0] + 2.0).abs().max()) == 0.0


@pytest.mark.parametrize("H,D,Dv,splits", [(3, 5, 7, [150]), (2, 32, 48, [70, 1, 1, 64, 3, 130]), (2, 130, 5, [64, 65])])
def test_matrix_memory_long_stretches_in_chunks(lib, H, D, Dv, splits):
    from oracle import zusuvik as O
    n = sum(splits)
    m, w, X = _memory_case(H, D, Dv, 8.0, 21, n, gate_gain=6.0)
    want, (S, nn, mm) = O.matrix_memory(X.double(), m, {k: v.double() for k, v in w.items()}, 1e-5)
    got, (state, mx) = _run_memory(lib, m, w, X, splits, torch.float32)
    assert close(got, 1.2 * want, F32_TOL) and close(state[2][:, :, :Dv], S, F32_TOL) and close(mx[2], mm, 1e-6)
    again, _ = _run_memory(lib, m, w, X, [1] * 30, torch.float32, state=(state, mx))      # the slot is used again from position 0
    assert close(again, 1.2 * want[:30], F32_TOL)


# ------------------------------------------------------------------ experts
@pytest.mark.parametrize("E,top,T", [(5, 2, 7), (3, 3, 1), (70, 4, 33), (16, 1, 5), (130, 8, 3)])
def test_routing_on_the_logits(lib, E, top, T):
    from oracle import zusuvik as O
    z = rnd((T, E + 1), 1, 3.0)                           # one more column behind the logits, as the shared expert's gate brings
    z[0, 1] = z[0, 0]                                     # a tie goes to the lower index
    if E > 4:
        z[-1, 3] = z[-1, 4] = z[-1].max() + 1.0
    sel, wt = zeros(T * top, dtype=torch.int32), zeros(T * top)
    call("umb_moe_route_top", sel, wt, dev(z), E + 1, T, E, top)
    s_want, w_want = O.route_top_logits(z[:, :E].double(), top)
    assert torch.equal(sel.view(T, top).cpu().long(), s_want) and close(wt.view(T, top), w_want, 1e-6)
    assert float((wt.view(T, top).sum(-1) - 1).abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,F,K,limit", [(1, 12, 8, 1.5), (5, 9, 6, 0.3), (37, 20, 32, 1.0), (300, 136, 72, 2.5)])
def test_linear_capped_gated_epilogue(lib, dtype, T, F, K, limit):
    """the limit binds on both sides for a good share of the values (inputs of unit scale against limits of 0.3 .. 2.5)"""
    x, wg, wu = rnd((T, K), 1).to(dtype), (2.0 * rnd((F, K), 2) / K ** 0.5).to(dtype), (2.0 * rnd((F, K), 3) / K ** 0.5).to(dtype)
    out = zeros(T, F, dtype=dtype)
    call("umb_seq_linear_glu", out, dev(x), dev(torch.cat([wg, wu])), None, T, 2 * F, K, limit, 1.702, code(dtype))
    g = (x.double() @ wg.double().T).clamp(max=limit)
    u = (x.double() @ wu.double().T).clamp(-limit, limit)
    assert float((g == limit).double().mean()) > 0.02 and float((u.abs() == limit).double().mean()) > 0.02
    assert close(out, g * torch.sigmoid(1.702 * g) * (u + 1), 1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shared", [True, False])
def test_expert_mixture_through_its_entry_points(lib, dtype, shared):
    from oracle import zusuvik as O
    T, W, E, top, F, Fs = 23, 24, 6, 3, 10, 7
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": F, "limit": 0.8}}
    w = {"router": 2.0 * rnd((E, W), 2) / W ** 0.5, "router.b": rnd((E,), 3, 0.5)}
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = rnd((F, W), 10 + e) / W ** 0.5 * 2, rnd((F, W), 30 + e) / W ** 0.5 * 2, rnd((W, F), 50 + e) / F ** 0.5
    if shared:
        mlp["shared"] = {"ff": Fs, "limit": 0.4}
        w.update({"shared.gate": 2 * rnd((Fs, W), 70) / W ** 0.5, "shared.up": 2 * rnd((Fs, W), 71) / W ** 0.5, "shared.down": rnd((W, Fs), 72) / Fs ** 0.5,
                  "shared.sg": 3 * rnd((1, W), 73) / W ** 0.5})
    w = {k: v.to(dtype) for k, v in w.items()}
    h = rnd((T, W), 1).to(dtype)
    want = O.expert_mixture(h.double(), mlp, {k: v.double() for k, v in w.items()})
    c, pairs, tiles = code(dtype), T * top, (T * top + 15) // 16 + E
    rw = torch.cat([w["router"]] + ([w["shared.sg"]] if shared else []))
    rb = torch.cat([w["router.b"]] + ([torch.zeros(1, dtype=dtype)] if shared else []))
    NR = rw.shape[0]
    logits = zeros(T, NR)
    call("umb_seq_linear", logits, dev(h), dev(rw), dev(rb), T, NR, W, 0, c)
    sel, wt, pos, tl = zeros(pairs, dtype=torch.int32), zeros(pairs), zeros(pairs, dtype=torch.int32), zeros(tiles, 3, dtype=torch.int32)
    xs, act, ye, y = zeros(pairs, W, dtype=dtype), zeros(pairs, F, dtype=dtype), zeros(pairs, W), zeros(T, W)
    if shared:
        sa = zeros(T, Fs, dtype=dtype)
        call("umb_seq_linear_glu", sa, dev(h), dev(torch.cat([w["shared.gate"], w["shared.up"]])), None, T, 2 * Fs, W, 0.4, 1.702, c)
        call("umb_seq_linear", y, sa, dev(w["shared.down"]), None, T, W, Fs, 0, c)
    call("umb_moe_route_top", sel, wt, logits, NR, T, E, top)
    call("umb_moe_plan", pos, tl, sel, T, E, top, tiles, 16)
    call("umb_moe_scatter", xs, dev(h), None, pos, T, W, top, c)
    gu = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)])
    call("umb_seq_linear_grouped_glu", act, xs, dev(gu), tl, tiles, 16, 2 * F * W, 2 * F, W, 0.8, 1.702, c)
    call("umb_seq_linear_grouped", ye, act, dev(torch.stack([w[f"e{e}.down"] for e in range(E)])), tl, tiles, 16, W * F, W, F, 0, c)
    call("umb_moe_combine_gated", y, y if shared else None, ye, wt, pos, _offset(logits, E) if shared else None, NR, T, W, top)
    assert close(y, want, 1e-5 if dtype == torch.float32 else 3e-2)


# ------------------------------------------------------------------ whole models
def _oracle_logits(cfgd, sd, toks, margins=None, per_layer=False):
    from oracle import zusuvik as O
    lg, layers, _ = O.forward(cfgd, sd, toks, margins=margins)
    return (lg, layers) if per_layer else lg


def _calm_tokens(cfgd, sd, n, dtype, seed0=5):
    """a token sequence whose expert choices stand clear of every runner-up (16-bit runs drift by a percent: a choice that
    hangs on less would make the test one of rounding, not of the mechanism) -> (tokens, the oracle's logits)"""
    for seed in range(seed0, seed0 + 200):
        toks, margins = tokens(n, cfgd["vocab"], seed), []
        want = _oracle_logits(cfgd, sd, toks, margins)
        if dtype == torch.float32 or not margins or min(margins) > 0.02:
            return toks, want
    raise AssertionError("no calm token sequence found")


def _few_experts(cfgd):
    """the same shape with at most six experts of which at most two are used (for 16-bit runs)"""
    out = json.loads(json.dumps(cfgd))
    for ly in out["layers"]:
        if ly["mlp"] and ly["mlp"]["router"]["experts"] > 8:
            ly["mlp"]["router"] = {"experts": 6, "top": 2}
    return out


def _all_experts(cfgd):
    """the same shape with four experts that are all used: among a thousand routing decisions of a long 16-bit run one is always
    a close call, so such runs keep the weights (softmax over the chosen logits) and drop the choice"""
    out = json.loads(json.dumps(cfgd))
    for ly in out["layers"]:
        if ly["mlp"]:
            ly["mlp"]["router"] = {"experts": 4, "top": 4}
    return out


@pytest.mark.parametrize("name", ["mixed", "odd", "plain", "wide"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_prefill_decode_portions_against_oracle(lib, name, dtype):
    from zusuvik_helpers import CONFIGS, build
    cfgd = CONFIGS[name] if dtype == torch.float32 else _few_experts(CONFIGS[name])
    m, sd = build(cfgd, dtype, seed=11, page=4)
    n = 41
    toks, want = _calm_tokens(cfgd, sd, n, dtype)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    m.open("w")
    whole, layers = m.forward_batch([("w", toks)], want=[list(range(n))], trace=True)
    whole = whole.clone()
    if dtype == torch.float32:                      # the residual after every layer run (a repeated layer counts every time)
        _, lo = _oracle_logits(cfgd, sd, toks, per_layer=True)
        assert layers.shape[0] == lo.shape[0] == len(m.config.layers) and close(layers, lo, F32_TOL)
    assert rel_err(whole, want) < tol
    same = F32_TOL if dtype == torch.float32 else 2e-2          # the model against itself under another schedule
    for sid, splits in (("d", [1] * n), ("p", [2, 2, 7, 1, 16, 3, 10]), ("q", [30] + [1] * 11), ("r", [17, 2, 2, 20])):
        m.open(sid)
        rows, at = [], 0
        for k in splits:
            rows.append(m.forward_batch([(sid, toks[at:at + k])], want=[list(range(k))]).clone())
            at += k
        got = torch.cat(rows)
        assert rel_err(got, want) < tol, (sid, "against the oracle")
        assert rel_err(got, whole) < same, (sid, "against the whole prompt")
        m.close(sid)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_unequal_batch_equals_each_alone(lib, dtype):
    """three requests of different lengths prefilled in one step and decoded together, the shortest ending first, against
    each of them alone; then a new request in the slot and pages the shortest one gave back"""
    from zusuvik_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    m, _ = build(cfgd, dtype, seed=3, page=4, batch=3)
    V = cfgd["vocab"]
    seqs = {"a": tokens(33, V, 1), "b": tokens(9, V, 2), "c": tokens(21, V, 3)}
    pre = {"a": 20, "b": 1, "c": 13}
    alone = {}
    for k, t in list(seqs.items()) + [("d", tokens(17, V, 4))]:
        m.open(k)
        alone[k] = m.forward_batch([(k, t)], want=[list(range(len(t)))]).clone()
        m.close(k)
    got = {k: [] for k in seqs}
    for k in seqs:
        m.open(k)
    out = m.forward_batch([(k, seqs[k][:pre[k]]) for k in seqs], want=[list(range(pre[k])) for k in seqs]).clone()
    at = 0
    for k in seqs:
        got[k].append(out[at:at + pre[k]])
        at += pre[k]
    done = dict(pre)
    live = list(seqs)
    while live:
        out = m.forward_batch([(k, [seqs[k][done[k]]]) for k in live], want=[[0]] * len(live)).clone()
        for i, k in enumerate(live):
            got[k].append(out[i:i + 1])
            done[k] += 1
        for k in [k for k in live if done[k] == len(seqs[k])]:
            m.close(k)
            live.remove(k)
            if k == "b":                              # its slot and pages are handed to a new request at once
                m.open("d")
                got["d"] = [m.forward_batch([("d", tokens(17, V, 4))], want=[list(range(17))]).clone()]
                m.close("d")
    tol = F32_TOL if dtype == torch.float32 else 2e-2
    for k in got:
        assert rel_err(torch.cat(got[k]), alone[k]) < tol, k


def test_model_long_decoding_and_first_tokens(lib):
    """fp32: 150 tokens decoded one by one after a two-token prompt (pages of 4 tokens used up and down the table, the ring of the
    convolution going round, the running maximum settling) against the oracle's whole-sequence pass"""
    from zusuvik_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    m, sd = build(cfgd, torch.float32, seed=7, page=4, batch=2, max_tokens=400)
    toks = tokens(152, cfgd["vocab"], seed=9)
    want = _oracle_logits(cfgd, sd, toks)
    m.open("x")
    rows = [m.forward_batch([("x", toks[:2])], want=[[0, 1]]).clone()]
    for t in toks[2:]:
        rows.append(m.forward_batch([("x", [t])], want=[[0]]).clone())
    got = torch.cat(rows)
    assert rel_err(got, want) < F32_TOL
    assert rel_err(got[:3], want[:3]) < F32_TOL


@pytest.mark.parametrize("name", ["mixed", "wide"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_long_prompt_in_one_step_and_in_portions(lib, name, dtype):
    """stretches long enough for the chunked scans and the matrix-pipe attention, cut at and beside chunk and page borders"""
    from zusuvik_helpers import CONFIGS, build
    cfgd = CONFIGS[name] if dtype == torch.float32 else _all_experts(CONFIGS[name])
    m, sd = build(cfgd, dtype, seed=5, page=16, batch=2, max_length=320, max_tokens=700)
    n = 200
    toks, want = _calm_tokens(cfgd, sd, n, dtype, seed0=40)
    m.open("w")
    whole = m.forward_batch([("w", toks)], want=[list(range(n))]).clone()

    def holds(got):
        if dtype == torch.float32:
            return rel_err(got, want) < F32_TOL
        # 16 bits through a stack this narrow: a row in a hundred lands several times the typical error away, under every
        # schedule alike (the schedules agree with one another far more closely, below)
        e = row_errs(got, want)
        return float(e.mean()) < 1.5e-2 and float(e.quantile(0.9)) < BF16_TOL and float(e.max()) < 0.2
    assert holds(whole)
    for sid, splits in (("p", [64, 65, 1, 1, 69]), ("q", [127, 2, 71])):
        m.open(sid)
        rows, at = [], 0
        for k in splits:
            rows.append(m.forward_batch([(sid, toks[at:at + k])], want=[list(range(k))]).clone())
            at += k
        assert holds(torch.cat(rows)), sid
        assert rel_err(torch.cat(rows), whole) < (F32_TOL if dtype == torch.float32 else 2e-2), sid
        m.close(sid)


def test_model_decode_steps_replayed_as_graphs_equal_eager_launches(lib):
    from zusuvik_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    V = cfgd["vocab"]
    seqs = {"a": tokens(30, V, 1), "b": tokens(24, V, 2)}
    outs = {}
    for graph in (False, True):
        m, _ = build(cfgd, torch.float32, seed=3, page=4, batch=2, hip_graph=graph)
        for k in seqs:
            m.open(k)
        rows = [m.forward_batch([(k, seqs[k][:10]) for k in seqs], want=[[9], [9]]).clone()]
        for i in range(10, 24):
            rows.append(m.forward_batch([(k, [seqs[k][i]]) for k in seqs], want=[[0], [0]]).clone())
            torch.cuda.synchronize()
        outs[graph] = torch.cat(rows)
    assert torch.equal(outs[False], outs[True])


def _engine(cfgd, dtype, sd=None, **kw):
    from zusuvik_helpers import build
    from umbrella_amd.speculation.auto_engine import AutoEngine
    from umbrella_amd.speculation.speculation_utils import IdTokenizer
    m, sd = build(cfgd, dtype, seed=21, page=4, batch=kw.pop("batch", 3), max_length=96, max_tokens=kw.pop("max_tokens", 512), sd=sd)
    e = AutoEngine.from_config("cuda:0", engine="batch", model="tiny", dtype=dtype, target_model_obj=m, tokenizer=IdTokenizer(), **kw)
    e.initialize()
    return e, sd


def _oracle_greedy(cfgd, sd, prompt, n):
    toks, margins = list(prompt), []
    for _ in range(n):
        row = _oracle_logits(cfgd, sd, toks)[-1]
        top = torch.topk(row, 2).values
        margins.append(float(top[0] - top[1]))
        toks.append(int(row.argmax()))
    return toks[len(prompt):], margins


def test_engine_greedy_generation_matches_oracle(lib):
    """five queued requests through the scheduler (three slots: two batches), greedy, fp32: the oracle's tokens"""
    from zusuvik_helpers import CONFIGS
    cfgd = CONFIGS["mixed"]
    e, sd = _engine(cfgd, torch.float32)
    prompts = [tokens(n, cfgd["vocab"], seed=n) for n in (7, 1, 12, 3, 9)]
    outs = e.generate_batch(prompts, max_new_tokens=10)
    for p, got in zip(prompts, outs):
        want, margins = _oracle_greedy(cfgd, sd, p, 10)
        k = next((i for i, (a, b) in enumerate(zip(got, want)) if a != b), None)
        assert k is None or margins[k] < 1e-4, (got, want, margins)
    assert not e.target_model.kv_cache.seqs and len(e.target_model.kv_cache.free_slots) == 3
    api = e.generate(input_ids=prompts[2], max_new_tokens=10)
    assert api["generated_tokens"] == outs[2]


def test_engine_sampling_is_seeded_and_in_range(lib):
    from zusuvik_helpers import CONFIGS
    cfgd = CONFIGS["odd"]
    e, _ = _engine(cfgd, torch.bfloat16, temperature=0.8, topk=8, topp=0.9, repetition_penalty=1.2, seed=5)
    prompts = [tokens(6, cfgd["vocab"], seed=1), tokens(11, cfgd["vocab"], seed=2)]
    a = e.generate_batch(prompts, max_new_tokens=12)
    e.reset()
    e.manual_seed(5)
    e.step_count.zero_()
    b = e.generate_batch(prompts, max_new_tokens=12)
    assert a == b and all(0 <= t < cfgd["vocab"] for o in a for t in o) and all(len(o) == 12 for o in a)


def test_trace_replay_command(lib, tmp_path):
    """bin/trace_run on a checkpoint directory: a mixed batch prefilled, decoded together, one request ending early"""
    import numpy as np
    from safetensors.torch import save_file
    from zusuvik_helpers import CONFIGS, checkpoint
    cfgd = CONFIGS["mixed"]
    _, sd = checkpoint(cfgd, seed=4)
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    mdir, out = tmp_path / "model", tmp_path / "out"
    mdir.mkdir()
    save_file({k: v.contiguous() for k, v in sd.items()}, str(mdir / "model.safetensors"))
    (mdir / "config.json").write_text(json.dumps(cfgd))
    V = cfgd["vocab"]
    a, b = tokens(26, V, 1), tokens(8, V, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:20], "want": [0, 19]}, {"id": "b", "tokens": b[:5], "want": [4]}],
              "end": []}]
    for i in range(6):
        ent = [{"id": "a", "tokens": [a[20 + i]], "want": [0]}]
        if 5 + i < len(b):
            ent.append({"id": "b", "tokens": [b[5 + i]], "want": [] if i == 1 else [0]})
        steps.append({"step": i + 1, "entries": ent, "end": (["b"] if 5 + i == len(b) - 1 else []) + (["a"] if i == 5 else [])})
    f32 = {k: v.float() for k, v in sd.items()}
    wa, wb = (_oracle_logits(cfgd, f32, t) for t in (a, b))
    for dt, tol in (("float32", F32_TOL), ("bfloat16", BF16_TOL)):
        p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(mdir), "--dtype", dt, "--out",
                            str(out), "--max-tokens", "64", "--page-size", "4"], input="\n".join(json.dumps(s) for s in steps),
                           capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-2000:]
        assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(7)]
        got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(3, V))
        assert rel_err(got0, torch.stack([wa[0], wa[19], wb[4]])) < tol
        got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(1, V))       # b wanted nothing in step 2
        assert rel_err(got2, wa[21:22]) < tol
        got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(2, V))
        assert rel_err(got3, torch.stack([wa[22], wb[7]])) < tol
        got6 = torch.from_numpy(np.fromfile(out / "6.f32", dtype="<f4").reshape(1, V))
        assert rel_err(got6, wa[25:26]) < tol
