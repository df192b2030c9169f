"""The Tomopel design on the HIP path against the plain oracle (oracle/tomopel.py): its mechanisms alone through their own
entry points of libumbrella_seq.so (residual streams, the minimal gated recurrence, the state-space layer on the general linear
scan, softmax attention with a distance bias, softmax routing with weighted outputs, the relu^2 epilogue), then whole models
through the runtime, the cache manager, the batch engine and the trace replay command.

fp32 runs are the sharp ones (every comparison to ~1e-5: one key too many, a bias one bucket off or a lost state is a
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


def close(got, want, tol):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30)) < tol


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).max())


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rnd(shape, seed, scale=1.0):
    return scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))


def code(dtype):
    from umbrella_amd import _lib
    return _lib.seq_dtype_code(dtype)


class Steps:
    """the index arrays of a step for sequences that each bring `counts[b]` rows from position `pos0[b]` in slot `slots[b]`"""

    def __init__(self, counts, pos0, slots):
        self.pos, self.slot, self.row0 = [], [], []
        for n, p, s in zip(counts, pos0, slots):
            self.row0.append(len(self.pos))
            self.pos += list(range(p, p + n))
            self.slot += [s] * n
        self.T, self.B = len(self.pos), len(counts)
        self.d = dict(pos=i32(self.pos), slot=i32(self.slot), seq_slot=i32(slots), seq_row0=i32(self.row0), seq_pos0=i32(pos0),
                      seq_len=i32(counts))


# ------------------------------------------------------------------ residual streams
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("S,W,T", [(1, 40, 3), (2, 300, 5), (3, 1500, 2), (5, 3000, 2), (2, 5000, 1), (8, 24, 4)])
def test_stream_embed_seam_read(lib, dtype, S, W, T):
    from oracle import tomopel as O
    from umbrella_amd import _lib
    V, eps, m, scale = 11, 1e-5, 0.6, 1.7
    embed = rnd((V, W), 1).to(dtype)
    w1, w2, wf = ((0.2 * rnd((W,), k)).to(dtype) for k in (2, 3, 4))
    tin, tin2 = rnd((S,), 5) + 1.0 / S, rnd((S,), 6) + 1.0 / S
    tout, tmix = rnd((S,), 7) + 1.0, torch.eye(S) + 0.3 * rnd((S, S), 8)
    toks = tokens(T, V, 9)
    y = rnd((T, W), 10)
    x = torch.zeros(T, S * W, dtype=torch.float32, device="cuda:0")
    h = torch.zeros(T, W, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_hc_embed", x, h, dev(embed), i32(toks), scale, dev(tin), dev(w1), 1.0, T, W, V, S, eps, code(dtype))
    xs = (embed.double()[toks] * scale)[None].repeat(S, 1, 1)
    want_h = O.offset_rms_norm(O.streams_read(xs, tin.double()), w1.double(), eps)
    tol = F32_TOL if dtype == torch.float32 else 1e-2
    assert close(x.view(T, S, W).transpose(0, 1), xs, 1e-6) and close(h, want_h, tol)
    _lib.seq_call("umb_hc_seam", x, h, dev(y), dev(tmix), dev(tout), m, dev(tin2), dev(w2), 1.0, T, W, S, eps, code(dtype))
    xs2 = O.streams_write(xs, y.double(), tmix.double(), tout.double(), m)
    assert close(x.view(T, S, W).transpose(0, 1), xs2, 1e-5)
    assert close(h, O.offset_rms_norm(O.streams_read(xs2, tin2.double()), w2.double(), eps), tol)
    # the last seam of a model writes only; the final read sums the streams of the gathered rows
    before = h.clone()
    _lib.seq_call("umb_hc_seam", x, None, dev(y), dev(tmix), dev(tout), m, None, None, 1.0, T, W, S, eps, code(dtype))
    xs3 = O.streams_write(xs2, y.double(), tmix.double(), tout.double(), m)
    assert close(x.view(T, S, W).transpose(0, 1), xs3, 1e-5) and torch.equal(h, before)
    rows = [T - 1, 0]
    u = torch.zeros(2, W, dtype=torch.float32, device="cuda:0")
    hf = torch.zeros(2, W, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_hc_read", u, hf, x, i32(rows), None, dev(wf), 1.0, 2, W, S, eps, code(dtype))
    assert close(u, xs3.sum(0)[rows], 1e-5) and close(hf, O.offset_rms_norm(xs3.sum(0)[rows], wf.double(), eps), tol)


def test_stream_seam_with_trivial_tables_is_the_plain_residual(lib):
    from oracle import tomopel as O
    from umbrella_amd import _lib
    T, W, m, eps = 3, 70, 0.5, 1e-6
    x0, y, w = rnd((T, W), 1), rnd((T, W), 2), 0.1 * rnd((W,), 3)
    x = dev(x0.clone())
    h = torch.zeros(T, W, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_hc_seam", x, h, dev(y), None, None, m, None, dev(w), 0.0, T, W, 1, eps, code(torch.float32))
    assert close(x, x0 + m * y, 1e-6) and close(h, O.unit_rms((x0 + m * y).double(), eps) * w.double(), F32_TOL)


# ------------------------------------------------------------------ minimal gated recurrence
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Wm,splits", [(24, [19]), (70, [1] * 12), (300, [2, 9, 1, 1, 17, 3]), (257, [40, 1, 1]),
                                       (70, [333]), (24, [129, 1, 200, 2, 131]), (300, [128, 160])])      # long stretches: pieces
def test_mingru_scan_prompt_portions_and_single_tokens(lib, dtype, Wm, splits):
    """the state is carried across steps; a second sequence in the batch with other lengths does not disturb it; the slot's old
    state is ignored by a sequence that starts at position 0"""
    from oracle import tomopel as O
    from umbrella_amd import _lib
    n = sum(splits)
    proj = rnd((n, 3 * Wm + 5), 1, 1.5)                                # wider than needed: a row stride of its own
    proj2 = rnd((n + 3, 3 * Wm + 5), 2, 1.5)
    eye = torch.eye(Wm, dtype=torch.float64)

    def oracle(p):                                                      # the projections are given: selection matrices as weights
        X = p.double()[:, 2:2 + 3 * Wm]
        zero = torch.zeros(Wm, Wm, dtype=torch.float64)
        sel = lambda k: torch.cat([eye if j == k else zero for j in range(3)], dim=1)      # noqa: E731
        none = torch.zeros(Wm, dtype=torch.float64)
        return O.min_gru(X, sel(0), none, sel(1), none, sel(2), eye)[0]
    state = torch.full((3, Wm), 1e6, dtype=torch.float32, device="cuda:0")       # loud leftovers in every slot
    got, got2, at, at2 = [], [], 0, 0
    for k, cnt in enumerate(splits):
        c2 = cnt + 3 if k == 0 else cnt                                 # the neighbour's portions are of other sizes
        both = torch.cat([proj2[at2:at2 + c2], proj[at:at + cnt]])
        st = Steps([c2, cnt], [at2, at], [0, 2])
        out = torch.zeros(st.T, Wm, dtype=dtype, device="cuda:0")
        need = _lib.load_seq().umb_mingru_scratch_floats(st.T, 2, Wm)
        scratch = torch.zeros(need, dtype=torch.float32, device="cuda:0")
        _lib.seq_call("umb_mingru_scan", out, state, dev(both), both.shape[1], 2, 2 + Wm, 2 + 2 * Wm, st.d["seq_slot"],
                      st.d["seq_row0"], st.d["seq_pos0"], st.d["seq_len"], 2, Wm, max(c2, cnt), scratch, need, code(dtype))
        got2.append(out[:c2].clone())
        got.append(out[c2:].clone())
        at, at2 = at + cnt, at2 + c2
    tol = F32_TOL if dtype == torch.float32 else 1e-2
    assert close(torch.cat(got), oracle(proj), tol) and close(torch.cat(got2), oracle(proj2), tol)


# ------------------------------------------------------------------ state-space layer
def _ssd_weights(width, H, Dv, N, G, taps, seed):
    inner, gn = H * Dv, G * N
    return dict(w_in=rnd((2 * inner + 2 * gn + H, width), seed) / width ** 0.5, conv_w=rnd((inner + 2 * gn, taps), seed + 1, 0.5),
                conv_b=rnd((inner + 2 * gn,), seed + 2, 0.3), dt_bias=rnd((H,), seed + 3, 0.5) - 1.0, a_log=rnd((H,), seed + 4, 0.5),
                d_skip=1.0 + rnd((H,), seed + 5, 0.2), norm_w=1.0 + rnd((inner,), seed + 6, 0.1))


def _run_ssd(lib, X, w, dtype, splits, H, Dv, N, G, NG, taps, eps, scale=1.0, slot=1, state=None, conv=None, col0=3, chunked=True):
    """prep + state ring + scan + gate through their entry points, the sequence cut into `splits`; returns the gated, normed
    rows [n, H Dv] (what the output projection reads)"""
    from umbrella_amd import _lib
    inner, gn = H * Dv, G * N
    C, lds = inner + 2 * gn, 2 * inner + 2 * gn
    proj_all = torch.cat([rnd((X.shape[0], col0), 77), (X.double() @ w["w_in"].double().T).float()], dim=1)    # junk columns in front
    ld = proj_all.shape[1]
    state = torch.full((3, H, N, Dv), 1e6, dtype=torch.float32, device="cuda:0") if state is None else state
    conv = torch.full((3, max(taps - 1, 1), C), 1e6, dtype=torch.float32, device="cuda:0") if conv is None else conv
    f32 = lambda k: dev(w[k], torch.float32)                             # noqa: E731
    outs, at = [], 0
    for cnt in splits:
        st = Steps([cnt], [at], [slot])
        proj = dev(proj_all[at:at + cnt])
        sx = torch.zeros(cnt, lds + 1, dtype=torch.float32, device="cuda:0")
        alpha = torch.zeros(cnt, H, dtype=torch.float32, device="cuda:0")
        la = torch.zeros(cnt, H, dtype=torch.float32, device="cuda:0")
        o = torch.zeros(cnt, inner, dtype=torch.float32, device="cuda:0")
        out = torch.zeros(cnt, inner + 2, dtype=dtype, device="cuda:0")
        single = int(cnt == 1)                                          # as the forward does: one launch for single tokens
        _lib.seq_call("umb_ssd_prep", sx, lds + 1, alpha, la, proj, ld, col0, dev(w["conv_w"], dtype), dev(w["conv_b"], dtype), conv,
                      f32("dt_bias"), f32("a_log"), st.d["pos"], st.d["slot"], cnt, H, Dv, G, N, taps, single, code(dtype))
        if not single:
            _lib.seq_call("umb_ssd_conv_update", conv, proj, ld, col0 + inner, st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
                          st.d["seq_len"], 1, C, taps)
        need = lib.umb_ssd_scan_chunked_floats(1, cnt, H, N, Dv) if cnt >= 64 and chunked else 0
        if need > 0:                                                    # as the forward does: long stretches in chunks
            scratch = torch.zeros(need, dtype=torch.float32, device="cuda:0")
            _lib.seq_call("umb_ssd_scan_chunked", o, state, sx[:, inner + gn:], lds + 1, sx[:, inner:], lds + 1, sx, lds + 1, la, G,
                          st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"], st.d["seq_len"], 1, cnt, H, N, Dv, scratch, need)
        else:
            _lib.seq_call("umb_lin_scan", o, state, sx[:, inner + gn:], lds + 1, sx[:, inner:], lds + 1, sx, lds + 1, alpha, 1, G,
                          st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"], st.d["seq_len"], 1, H, N, Dv, 1.0)
        _lib.seq_call("umb_ssd_gate", out, inner + 2, o, sx, lds + 1, C, proj, ld, col0, f32("d_skip"), dev(w["norm_w"], dtype), cnt, H,
                      Dv, NG, eps, scale, code(dtype))
        outs.append(out[:, :inner].clone())
        at += cnt
    return torch.cat(outs)


def _ssd_oracle(X, w, dtype, H, Dv, N, G, NG, eps):
    from oracle import tomopel as O
    r = (lambda t: t.to(dtype).double()) if dtype != torch.float32 else (lambda t: t.double())
    eye = torch.eye(H * Dv, dtype=torch.float64)
    return O.ssd(X.double(), w["w_in"].double(), r(w["conv_w"]), r(w["conv_b"]), w["dt_bias"].double(), w["a_log"].double(),
                 w["d_skip"].double(), r(w["norm_w"]), eye, heads=H, vdim=Dv, state=N, groups=G, norm_groups=NG, eps=eps)[0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,Dv,N,G,NG,taps", [(3, 4, 5, 1, 1, 3), (4, 6, 7, 2, 2, 2), (2, 5, 3, 1, 1, 1), (6, 8, 16, 3, 3, 5),
                                              (4, 32, 64, 2, 4, 4), (2, 20, 130, 1, 2, 3)])
def test_state_space_prompt_portions_and_single_tokens(lib, dtype, H, Dv, N, G, NG, taps):
    n, width, eps = 37, 24, 1e-5
    w = _ssd_weights(width, H, Dv, N, G, taps, seed=H + N)
    X = rnd((n, width), 5)
    want = _ssd_oracle(X, w, dtype, H, Dv, N, G, NG, eps)
    tol = F32_TOL if dtype == torch.float32 else 2e-2
    for splits in ([n], [1] * n, [2, 2, 7, 1, 16, 3, 6], [30] + [1] * 7, [1, 2, 3, 4, 27]):
        got = _run_ssd(lib, X, w, dtype, splits, H, Dv, N, G, NG, taps, eps)
        assert close(got, want, tol), splits
    assert close(_run_ssd(lib, X, w, dtype, [n], H, Dv, N, G, NG, taps, eps, scale=0.25), 0.25 * want, tol)


@pytest.mark.parametrize("H,Dv,N,G,NG,taps", [(3, 4, 5, 1, 1, 3), (4, 32, 64, 2, 4, 4), (2, 20, 130, 1, 2, 3), (2, 70, 16, 2, 1, 2),
                                              (1, 136, 24, 1, 1, 4)])
def test_state_space_long_stretches_in_chunks(lib, H, Dv, N, G, NG, taps):
    """stretches of 64 tokens and more take the chunked form (whole and partial chunks, a carried state in front, single tokens
    behind); against the oracle and against the token-by-token scan"""
    n, width, eps = 210, 24, 1e-5
    w = _ssd_weights(width, H, Dv, N, G, taps, seed=H + N)
    w["dt_bias"] = w["dt_bias"] - 1.5                                   # slow decays: the state remembers across chunks
    X = rnd((n, width), 5)
    want = _ssd_oracle(X, w, torch.float32, H, Dv, N, G, NG, eps)
    serial = _run_ssd(lib, X, w, torch.float32, [n], H, Dv, N, G, NG, taps, eps, chunked=False)
    assert close(serial, want, F32_TOL)
    for splits in ([n], [64, 146], [3, 128, 65, 1, 1, 12], [100, 1, 109], [65] + [1] * 81 + [64]):
        got = _run_ssd(lib, X, w, torch.float32, splits, H, Dv, N, G, NG, taps, eps)
        assert close(got, want, F32_TOL) and close(got, serial, F32_TOL), splits
    assert close(_run_ssd(lib, X, w, torch.bfloat16, [n], H, Dv, N, G, NG, taps, eps), _ssd_oracle(X, w, torch.bfloat16, H, Dv, N, G, NG, eps), 2e-2)


def test_state_space_slot_is_reused_without_leaking(lib):
    """a loud sequence leaves its state and convolution ring in the slot; the next one starts from zero"""
    H, Dv, N, G, NG, taps, eps = 3, 4, 5, 1, 1, 4, 1e-5
    w = _ssd_weights(24, H, Dv, N, G, taps, seed=3)
    state = torch.zeros(3, H, N, Dv, dtype=torch.float32, device="cuda:0")
    conv = torch.zeros(3, taps - 1, H * Dv + 2 * G * N, dtype=torch.float32, device="cuda:0")
    _run_ssd(lib, 30.0 * rnd((9, 24), 1), w, torch.float32, [9], H, Dv, N, G, NG, taps, eps, state=state, conv=conv)
    assert float(state[1].abs().max()) > 1.0
    X = rnd((11, 24), 2)
    got = _run_ssd(lib, X, w, torch.float32, [1, 1, 1, 8], H, Dv, N, G, NG, taps, eps, state=state, conv=conv)
    assert close(got, _ssd_oracle(X, w, torch.float32, H, Dv, N, G, NG, eps), F32_TOL)


def test_gated_linear_attention_still_runs_on_the_general_scan(lib):
    """umb_gla_scan is now one placement of umb_lin_scan: a decay per key channel, a q / k group per head"""
    from umbrella_amd import _lib
    H, D, Dv, n = 2, 12, 8, 21
    proj, alpha = rnd((n, 2 * H * D + H * Dv), 1), torch.sigmoid(rnd((n, H * D), 2) + 2.0)
    S = torch.zeros(H, D, Dv, dtype=torch.float64)
    want = torch.zeros(n, H, Dv, dtype=torch.float64)
    q, k, v = (proj.double()[:, a:b].reshape(n, H, -1) for a, b in ((0, H * D), (H * D, 2 * H * D), (2 * H * D, 2 * H * D + H * Dv)))
    al = alpha.double().reshape(n, H, D)
    for t in range(n):
        for h in range(H):
            S[h] = al[t, h][:, None] * S[h] + torch.outer(k[t, h], v[t, h])
            want[t, h] = S[h].T @ (q[t, h] * 0.5)
    st = Steps([n], [0], [0])
    o = torch.zeros(n, H * Dv, dtype=torch.float32, device="cuda:0")
    state = torch.zeros(1, H, D, Dv, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_gla_scan", o, state, dev(proj), proj.shape[1], dev(alpha), st.d["seq_slot"], st.d["seq_row0"], st.d["seq_pos0"],
                  st.d["seq_len"], 1, H, D, Dv, 0.5)
    assert close(o, want.reshape(n, -1), F32_TOL) and close(state[0], S, F32_TOL)


# ------------------------------------------------------------------ attention with a distance bias
def _attn_weights(width, H, G, D, E, rows, seed):
    return dict(wq=rnd((H * D, width), seed) / width ** 0.5, wk=rnd((G * D, width), seed + 1) / width ** 0.5,
                wv=rnd((G * E, width), seed + 2) / width ** 0.5, wg=rnd((H, width), seed + 3) / width ** 0.5,
                q_norm=1.0 + rnd((D,), seed + 4, 0.1), k_norm=1.0 + rnd((D,), seed + 5, 0.1), rel=rnd((rows, H), seed + 6, 0.8))


def _run_attn(lib, X, w, dtype, splits, H, G, D, E, scale, far, temp, eps, page=4, cache=None, seq="s", out_scale=1.0, window=2 ** 30,
              max_len=512, split_keys=True):
    """prep + attend through their entry points over a cache handed out by the cache manager -> [n, H E]"""
    from umbrella_amd import _lib
    from umbrella_amd.attn.cache import PagedSeqCache
    from umbrella_amd.models.tomopel import bias_by_distance
    if cache is None:
        cache = PagedSeqCache([(G, D, 0, E)], [], max_tokens=max_len, max_seqs=2, device="cuda:0", dtype=dtype, page=page)
    cache.open(seq)
    kv = cache.struct(0)
    r = lambda t: t.to(dtype).float()                                   # noqa: E731
    W_all = torch.cat([w["wq"], w["wk"], w["wv"], w["wg"]])
    proj_all = (X.double() @ W_all.double().T).float()
    ld = proj_all.shape[1]
    bias = dev(bias_by_distance(r(w["rel"]), far, max_len)) if w.get("rel") is not None else None
    outs, at = [], 0
    for cnt in splits:
        p0 = cache.extend(seq, cnt)
        st = Steps([cnt], [p0], [cache.slot(seq)])
        proj = dev(proj_all[at:at + cnt])
        q = torch.zeros(cnt, H * D, dtype=torch.float32, device="cuda:0")
        out = torch.zeros(cnt, H * E + 3, dtype=dtype, device="cuda:0")
        _lib.seq_call("umb_bsa_prep", q, kv, proj, ld, dev(w["q_norm"], dtype), dev(w["k_norm"], dtype), st.d["pos"], st.d["slot"], cnt,
                      H, G, D, E, temp[0], temp[1], eps, code(dtype))
        nd = bias.shape[1] if bias is not None else 0
        if cnt >= 16 and lib.umb_bsa_attend_tiled_ok(H, G, D, E, code(dtype)):       # as the forward chooses: the matrix pipe
            _lib.seq_call("umb_bsa_attend_tiled", out, H * E + 3, q, kv, proj, ld, H * D + G * D + G * E, bias, nd, st.d["seq_slot"],
                          st.d["seq_row0"], st.d["seq_pos0"], st.d["seq_len"], 1, cnt, H, G, D, E, window, scale, out_scale, 0.0, code(dtype))
        else:
            # steps of few rows with scratch: the keys of a row are dealt to several workgroups and merged
            need = cnt * H * 16 * (E + 2) if split_keys else 0
            scratch = torch.zeros(max(need, 1), dtype=torch.float32, device="cuda:0") if split_keys else None
            _lib.seq_call("umb_bsa_attend", out, H * E + 3, q, kv, proj, ld, H * D + G * D + G * E, bias, nd, st.d["pos"],
                          st.d["slot"], cnt, H, G, D, E, window, scale, out_scale, 0.0, scratch, need, code(dtype))
        assert float(out[:, H * E:].abs().max()) == 0.0
        outs.append(out[:, :H * E].clone())
        at += cnt
    return torch.cat(outs), cache


def _attn_oracle(X, w, dtype, H, G, D, E, scale, far, temp, eps):
    from oracle import tomopel as O
    r = (lambda t: t.to(dtype).double()) if dtype != torch.float32 else (lambda t: t.double())
    eye = torch.eye(H * E, dtype=torch.float64)
    return O.biased_attention(X.double(), w["wq"].double(), w["wk"].double(), w["wv"].double(), w["wg"].double(), eye, r(w["q_norm"]),
                              r(w["k_norm"]), r(w["rel"]), H=H, G=G, D=D, E=E, scale=scale, far=far, temp_coef=temp[0],
                              temp_every=max(temp[1], 1), eps=eps)[0]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,rows,far,temp", [(4, 2, 8, 6, 12, 40, (0.3, 8)), (3, 1, 7, 9, 4, 9, (0.0, 0)), (2, 2, 16, 16, 7, 25, (0.5, 1)),
                                                   (8, 2, 32, 64, 32, 70, (0.2, 16)), (6, 3, 24, 130, 9, 1000, (0.1, 5)),
                                                   (12, 1, 40, 48, 10, 33, (0.2, 7)), (4, 4, 136, 144, 6, 20, (0.0, 0)),
                                                   (2, 1, 16, 400, 8, 30, (0.1, 9)),
                                                   (1, 1, 8, 200, 16, 16, (1.0, 64))])
def test_biased_attention_prompt_portions_and_single_tokens(lib, dtype, H, G, D, E, rows, far, temp):
    """every bucket of the table is reached (far < n for most shapes), the temperature steps several times, keys sit on both
    sides of every page border (pages of 4)"""
    n, width, eps, scale = 90, 24, 1e-5, 0.4
    w = _attn_weights(width, H, G, D, E, rows, seed=H + D)
    X = rnd((n, width), 6)
    want = _attn_oracle(X, w, dtype, H, G, D, E, scale, far, temp, eps)
    tol = F32_TOL if dtype == torch.float32 else 2e-2
    for splits in ([n], [1] * n, [2, 2, 7, 1, 16, 3, 59], [70] + [1] * 20, [17, 2, 2, 69]):
        got, _ = _run_attn(lib, X, w, dtype, splits, H, G, D, E, scale, far, temp, eps)
        assert close(got, want, tol), splits
    got, _ = _run_attn(lib, X, w, dtype, [40] + [1] * 50, H, G, D, E, scale, far, temp, eps, split_keys=False)
    assert close(got, want, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_biased_attention_bucket_edges_show(lib, dtype):
    """the table is flat except for ONE loud row: a query sees the loud bias exactly for the distances of that bucket, so a key
    one position inside or outside the bucket's edge changes the output by much; checked for every bucket in turn, in a
    prompt and token by token"""
    from oracle import tomopel as O
    H, G, D, E, rows, far, n, width, eps, scale = 2, 1, 8, 8, 10, 30, 45, 16, 1e-5, 0.3
    X = rnd((n, width), 1)
    for loud in range(rows):
        w = _attn_weights(width, H, G, D, E, rows, seed=4)
        w["rel"] = torch.zeros(rows, H)
        w["rel"][loud] = 6.0
        want = _attn_oracle(X, w, dtype, H, G, D, E, scale, far, (0.0, 0), eps)
        tol = F32_TOL if dtype == torch.float32 else 2e-2
        for splits in ([n], [20] + [1] * 25):
            got, _ = _run_attn(lib, X, w, dtype, splits, H, G, D, E, scale, far, (0.0, 0), eps, page=8)
            assert close(got, want, tol), (loud, splits)
    edges = [d for d in range(1, n) if O.distance_bucket(d, rows, far) != O.distance_bucket(d - 1, rows, far)]
    assert len(edges) == rows - 1                                       # every bucket has an edge below n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_biased_attention_finds_one_far_key_among_hundreds(lib, dtype):
    """one early key is made to match the last queries (scaled so its score stands out): the output must be that key's value,
    in a prompt, in portions, and decoded; page borders of 64"""
    H, G, D, E, rows, far, n, width, eps, scale = 4, 2, 16, 16, 8, 50, 700, 32, 1e-6, 2.0
    w = _attn_weights(width, H, G, D, E, rows, seed=9)
    X = rnd((n, width), 2)
    X[3] = 0.0
    X[3, 0] = 40.0                                                      # a key direction of its own
    for t in range(n - 6, n):
        X[t] = X[3] + 0.01 * X[t]                                       # the last queries look for it
    want = _attn_oracle(X[:, :], w, dtype, H, G, D, E, scale, far, (0.3, 64), eps)
    tol = F32_TOL if dtype == torch.float32 else 2e-2
    for splits in ([n], [n - 8] + [1] * 8, [300, 394, 2, 2, 2]):
        got, _ = _run_attn(lib, X, w, dtype, splits, H, G, D, E, scale, far, (0.3, 64), eps, page=64, max_len=1024)
        assert close(got[-8:], want[-8:], tol), splits
        assert close(got[::50], want[::50], tol), splits


def test_biased_attention_pages_are_reused_without_leaking(lib):
    from umbrella_amd.attn.cache import PagedSeqCache
    H, G, D, E, rows, far, width, eps, scale = 3, 1, 8, 6, 6, 12, 20, 1e-5, 0.3
    w = _attn_weights(width, H, G, D, E, rows, seed=2)
    cache = PagedSeqCache([(G, D, 0, E)], [], max_tokens=40, max_seqs=1, device="cuda:0", dtype=torch.float32, page=4)
    _run_attn(lib, 50.0 * rnd((37, width), 1), w, torch.float32, [37], H, G, D, E, scale, far, (0.2, 4), eps, cache=cache, seq="one")
    first = list(cache.seqs["one"]["pages"])
    cache.close("one")
    X2 = rnd((30, width), 2)
    got, _ = _run_attn(lib, X2, w, torch.float32, [3, 1, 1, 25], H, G, D, E, scale, far, (0.2, 4), eps, cache=cache, seq="two")
    assert cache.seqs["two"]["pages"] == first[:len(cache.seqs["two"]["pages"])]
    assert close(got, _attn_oracle(X2, w, torch.float32, H, G, D, E, scale, far, (0.2, 4), eps), F32_TOL)


# ------------------------------------------------------------------ routing and the relu^2 experts
@pytest.mark.parametrize("E,top,T", [(5, 2, 7), (3, 3, 1), (70, 4, 33), (16, 1, 5), (130, 8, 3)])
def test_softmax_routing_with_correction(lib, E, top, T):
    from umbrella_amd import _lib
    logits, corr = rnd((T, E), E, 2.0), rnd((E,), top, 0.3)
    sel = torch.zeros(T, top, dtype=torch.int32, device="cuda:0")
    wt = torch.zeros(T, top, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_moe_route_softmax", sel, wt, dev(logits), dev(corr), T, E, top)
    s = torch.softmax(logits.double(), -1)
    order = torch.argsort(-(s + corr.double()), dim=-1, stable=True)[:, :top]
    assert torch.equal(sel.cpu().long(), order)
    chosen = torch.gather(s, 1, order)
    assert close(wt, chosen / chosen.sum(-1, keepdim=True), 1e-5)
    # without the correction the plain scores decide
    _lib.seq_call("umb_moe_route_softmax", sel, wt, dev(logits), None, T, E, top)
    assert torch.equal(sel.cpu().long(), torch.argsort(-s, dim=-1, stable=True)[:, :top])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,N,K", [(1, 12, 8), (5, 9, 6), (37, 20, 32), (300, 136, 72)])
def test_linear_relu_squared_epilogue(lib, dtype, T, N, K):
    from umbrella_amd import _lib
    x, w = rnd((T, K), 1).to(dtype), (rnd((N, K), 2) / K ** 0.5).to(dtype)
    out = torch.zeros(T, N, dtype=dtype, device="cuda:0")
    _lib.seq_call("umb_seq_linear", out, dev(x), dev(w), None, T, N, K, 4, code(dtype))
    assert close(out, torch.relu(x.double() @ w.double().T).pow(2), 1e-5 if dtype == torch.float32 else 2e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_weighted_combine_of_expert_outputs(lib, dtype):
    """plan + unweighted scatter + grouped relu^2 products + weighted combine against the oracle's routed feed-forward"""
    from oracle import tomopel as O
    from umbrella_amd import _lib
    T, W, E, top, F = 23, 24, 6, 3, 10
    h = rnd((T, W), 1).to(dtype)
    wr, corr = (2.0 * rnd((E, W), 2) / W ** 0.5).to(dtype), rnd((E,), 3, 0.1)
    ups, downs = (rnd((E, F, W), 4) / W ** 0.5).to(dtype), (rnd((E, W, F), 5) / F ** 0.5).to(dtype)
    want = O.routed_ff(h.double(), wr.double(), corr.double(), [(ups[e].double(), downs[e].double()) for e in range(E)], top)
    c, pairs, tiles = code(dtype), T * top, (T * top + 15) // 16 + E
    logits = torch.zeros(T, E, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_seq_linear", logits, dev(h), dev(wr), None, T, E, W, 0, c)
    sel, wt = torch.zeros(pairs, dtype=torch.int32, device="cuda:0"), torch.zeros(pairs, dtype=torch.float32, device="cuda:0")
    pos, tl = torch.zeros(pairs, dtype=torch.int32, device="cuda:0"), torch.zeros(tiles, 3, dtype=torch.int32, device="cuda:0")
    xs, act = torch.zeros(pairs, W, dtype=dtype, device="cuda:0"), torch.zeros(pairs, F, dtype=dtype, device="cuda:0")
    ye, y = torch.zeros(pairs, W, dtype=torch.float32, device="cuda:0"), torch.zeros(T, W, dtype=torch.float32, device="cuda:0")
    _lib.seq_call("umb_moe_route_softmax", sel, wt, logits, dev(corr), T, E, top)
    _lib.seq_call("umb_moe_plan", pos, tl, sel, T, E, top, tiles, 16)
    _lib.seq_call("umb_moe_scatter", xs, dev(h), None, pos, T, W, top, c)
    _lib.seq_call("umb_seq_linear_grouped", act, xs, dev(ups), tl, tiles, 16, F * W, F, W, 4, c)
    _lib.seq_call("umb_seq_linear_grouped", ye, act, dev(downs), tl, tiles, 16, W * F, W, F, 0, c)
    _lib.seq_call("umb_moe_combine_weighted", y, ye, wt, pos, T, W, top, 0)
    assert close(y, want, 1e-5 if dtype == torch.float32 else 3e-2)


# ------------------------------------------------------------------ whole models
def _oracle_logits(cfgd, sd, toks, margins=None, per_layer=False):
    from oracle import tomopel as O
    return O.forward(cfgd, sd, toks, margins=margins, per_layer=per_layer)


def _calm_tokens(cfgd, sd, n, dtype, seed0=5):
    """a token sequence whose expert choices stand clear of every runner-up (16-bit runs drift by a percent: a choice that
    hangs on less would make the test one of rounding, not of the mechanism) -> (tokens, the oracle's logits)"""
    for seed in range(seed0, seed0 + 200):
        toks, margins = tokens(n, cfgd["vocab"], seed), []
        want = _oracle_logits(cfgd, sd, toks, margins)
        if dtype == torch.float32 or not margins or min(margins) > 0.01:
            return toks, want
    raise AssertionError("no calm token sequence found")


def _few_experts(cfgd):
    """the same shape with at most six experts of which at most two are used (for 16-bit runs)"""
    out = json.loads(json.dumps(cfgd))
    for ly in out["layers"]:
        if ly["mlp"] and ly["mlp"]["kind"] == "moe" and ly["mlp"]["router"]["experts"] > 8:
            ly["mlp"]["router"] = {"experts": 6, "top": 2}
    return out


@pytest.mark.parametrize("name", ["mixed", "odd", "single", "wide"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_prefill_decode_portions_against_oracle(lib, name, dtype):
    from tomopel_helpers import BIAS_ROWS, CONFIGS, build
    cfgd = CONFIGS[name] if dtype == torch.float32 else _few_experts(CONFIGS[name])
    m, sd = build(cfgd, dtype, seed=11, page=4, bias_rows=BIAS_ROWS[name])
    n = 41
    toks, want = _calm_tokens(cfgd, sd, n, dtype)
    tol = F32_TOL if dtype == torch.float32 else BF16_TOL
    m.open("w")
    whole, layers = m.forward_batch([("w", toks)], want=[list(range(n))], trace=True)
    whole = whole.clone()
    if dtype == torch.float32:                      # the sum of the residual streams after every layer
        _, lo = _oracle_logits(cfgd, sd, toks, per_layer=True)
        assert layers.shape[0] == len(cfgd["layers"]) and close(layers, lo, F32_TOL)
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


def test_model_without_stream_weights_is_the_plain_residual(lib):
    from tomopel_helpers import CONFIGS, build
    cfgd = json.loads(json.dumps(CONFIGS["single"]))
    del cfgd["streams"]
    m, sd = build(cfgd, torch.float32, seed=2, bias_rows=6, stream_weights=False)
    assert not any(".hc" in k for k in sd)
    toks = tokens(19, cfgd["vocab"], 3)
    m.open("a")
    got = m.forward_batch([("a", toks)], want=[list(range(19))])
    assert rel_err(got, _oracle_logits(cfgd, sd, toks)) < F32_TOL


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_model_unequal_batch_equals_each_alone(lib, dtype):
    """three requests of different lengths prefilled in one step and decoded together, the shortest ending first, against
    each of them alone; then a new request in the slot and pages the shortest one gave back"""
    from tomopel_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    m, _ = build(cfgd, dtype, seed=3, page=4, batch=3, bias_rows=12)
    V = cfgd["vocab"]
    seqs = {"a": tokens(33, V, 1), "b": tokens(9, V, 2), "c": tokens(21, V, 3)}
    pre = {"a": 20, "b": 1, "c": 13}
    alone = {}
    for k, t in seqs.items():
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
    late = None
    while any(done[k] < len(seqs[k]) for k in seqs):
        live = [k for k in seqs if done[k] < len(seqs[k])]
        out = m.forward_batch([(k, [seqs[k][done[k]]]) for k in live], want=[[0]] * len(live)).clone()
        for i, k in enumerate(live):
            got[k].append(out[i:i + 1])
            done[k] += 1
            if done[k] == len(seqs[k]):
                m.close(k)
                if k == "b":                            # its slot and pages go to a newcomer while a and c go on
                    late = tokens(15, V, 4)
                    seqs["z"], done["z"], got["z"] = late, 0, []
                    m.open("z")
                    assert m.kv_cache.slot("z") == 1
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    m.open("z0")
    alone["z"] = m.forward_batch([("z0", late)], want=[list(range(len(late)))]).clone()
    for k in seqs:
        assert rel_err(torch.cat(got[k]), alone[k]) < tol, k


def test_model_long_decoding_and_first_tokens(lib):
    """fp32: 150 tokens decoded one by one after a two-token prompt (every bias bucket passed, the temperature stepping, pages
    of 4 tokens used up and down the table) against the oracle's whole-sequence pass"""
    from tomopel_helpers import CONFIGS, build
    cfgd = CONFIGS["mixed"]
    m, sd = build(cfgd, torch.float32, seed=7, page=4, batch=2, max_tokens=400, bias_rows=12)
    toks = tokens(152, cfgd["vocab"], seed=9)
    want = _oracle_logits(cfgd, sd, toks)
    m.open("x")
    rows = [m.forward_batch([("x", toks[:2])], want=[[0, 1]]).clone()]
    for t in toks[2:]:
        rows.append(m.forward_batch([("x", [t])], want=[[0]]).clone())
    got = torch.cat(rows)
    assert rel_err(got, want) < F32_TOL
    assert rel_err(got[:3], want[:3]) < F32_TOL


@pytest.mark.parametrize("name", ["mixed", "single"])
def test_model_long_prompt_in_one_step_and_in_portions(lib, name):
    """fp32: a 200-token prompt (state-space chunks of 64, minGRU pieces from 128 tokens on, matrix-free attention) whole, in two
    long portions, and with a second sequence of another length beside it, against the oracle"""
    from tomopel_helpers import BIAS_ROWS, CONFIGS, build
    cfgd = CONFIGS[name]
    m, sd = build(cfgd, torch.float32, seed=13, page=4, batch=3, max_tokens=1200, max_length=512, bias_rows=BIAS_ROWS[name])
    toks, other = tokens(200, cfgd["vocab"], 21), tokens(77, cfgd["vocab"], 22)
    want, want2 = _oracle_logits(cfgd, sd, toks), _oracle_logits(cfgd, sd, other)
    rows = list(range(0, 200, 7)) + [199]
    m.open("a")
    assert rel_err(m.forward_batch([("a", toks)], want=[rows]), want[rows]) < F32_TOL
    m.open("b")
    first = m.forward_batch([("b", toks[:130])], want=[[r for r in rows if r < 130]]).clone()
    second = m.forward_batch([("b", toks[130:])], want=[[r - 130 for r in rows if r >= 130]]).clone()
    assert rel_err(torch.cat([first, second]), want[rows]) < F32_TOL
    m.close("a"), m.close("b")
    m.open("c"), m.open("d")
    both = m.forward_batch([("c", other), ("d", toks)], want=[[76], rows])
    assert rel_err(both[:1], want2[76:77]) < F32_TOL and rel_err(both[1:], want[rows]) < F32_TOL


def test_model_decode_steps_replayed_as_graphs_equal_eager_launches(lib):
    from tomopel_helpers import CONFIGS, build
    from umbrella_amd.models import tomopel
    cfgd = CONFIGS["mixed"]
    m, sd = build(cfgd, torch.float32, seed=5, page=4, batch=2, bias_rows=12)
    g = tomopel.Tomopel("tiny", batch_size=2, max_length=256, max_tokens=1024, device="cuda:0", dtype=torch.float32, state_dict=sd,
                        config=tomopel.config_from_dict(cfgd), page_size=4, hip_graph=True)
    g.alloc()
    toks = tokens(30, cfgd["vocab"], 1)
    for mm in (m, g):
        mm.open("a")
        mm.forward_batch([("a", toks[:10])])
    for t in toks[10:]:
        a = m.forward_batch([("a", [t])]).clone()
        torch.cuda.synchronize()
        b = g.forward_batch([("a", [t])]).clone()
        assert torch.equal(a, b)


def test_cache_runs_out_loudly_and_recovers(lib):
    from tomopel_helpers import CONFIGS, build
    cfgd = CONFIGS["odd"]
    m, _ = build(cfgd, torch.bfloat16, page=4, batch=2, max_tokens=16, bias_rows=4)
    m.open("a")
    with pytest.raises(RuntimeError):
        m.forward_batch([("a", tokens(40, cfgd["vocab"], 1))])
    m.close("a")
    m.open("b")
    assert m.forward_batch([("b", tokens(10, cfgd["vocab"], 2))]).shape == (1, cfgd["vocab"])


# ------------------------------------------------------------------ engine and command line
def _engine(cfgd, dtype, sd=None, bias_rows=16, **kw):
    from tomopel_helpers import build
    from umbrella_amd.speculation.auto_engine import AutoEngine
    from umbrella_amd.speculation.speculation_utils import IdTokenizer
    m, sd = build(cfgd, dtype, seed=21, page=4, batch=kw.pop("batch", 3), max_length=96, max_tokens=kw.pop("max_tokens", 512), sd=sd,
                  bias_rows=bias_rows)
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
    from tomopel_helpers import CONFIGS
    cfgd = CONFIGS["mixed"]
    e, sd = _engine(cfgd, torch.float32, bias_rows=12)
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
    from tomopel_helpers import CONFIGS
    cfgd = CONFIGS["odd"]
    e, _ = _engine(cfgd, torch.bfloat16, bias_rows=4, temperature=0.8, topk=8, topp=0.9, repetition_penalty=1.2, seed=5)
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
    from tomopel_helpers import CONFIGS, checkpoint
    cfgd = CONFIGS["mixed"]
    _, sd = checkpoint(cfgd, seed=4, bias_rows=12)
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
