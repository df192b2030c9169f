"""CPU-side checks of the sequence-mixer family: the design's config reader and tensor table, the page / slot manager,
the batch engine's scheduler (with a stand-in model), the oracle's own visibility rules, and the library's ABI."""
import json
import os
import re

import pytest
import torch

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))


def test_config_reader_keeps_every_size_and_constant(tmp_path):
    from seqmix_helpers import CONFIGS
    from umbrella_amd.models import gitopel
    from umbrella_amd.models.auto_model import AutoModelLM
    from umbrella_amd.models.config import read_architecture
    cfgd = CONFIGS["wide_pool"]
    (tmp_path / "config.json").write_text(json.dumps(cfgd))
    cfg = gitopel.config_from_dir(str(tmp_path))
    assert (cfg.vocab_size, cfg.width, cfg.norm_groups, cfg.norm_eps) == (130, 72, 3, 1e-5)
    a0, a1, g2 = (ly.mixer for ly in cfg.layers)
    assert (a0.heads, a0.kv_heads, a0.dim, a0.window, a0.pool, a0.rot_dims, a0.scale) == (2, 1, 32, 9, 7, 32, 0.3)
    assert (a1.heads, a1.kv_heads, a1.dim, a1.window, a1.pool, a1.rot_dims) == (6, 3, 8, 4, 11, 0)
    assert (g2.kind, g2.heads, g2.dim, g2.vdim, g2.tau) == ("gla", 2, 16, 8, 8.0)
    assert [ly.ff for ly in cfg.layers] == [56, 0, 16]
    assert read_architecture(str(tmp_path)) == "Gitopel"
    assert AutoModelLM._ARCHITECTURE_MAPPING["Gitopel"] is gitopel.Gitopel
    shapes = gitopel.tensor_shapes(cfg, rank=5)
    assert shapes["l0.mix.q"] == (64, 72) and shapes["l0.mix.k"] == (32, 72) and shapes["l0.mix.g"] == (2, 72)
    assert shapes["l2.mix.a1"] == (5, 72) and shapes["l2.mix.a2"] == (32, 5) and shapes["l2.mix.norm"] == (8,)
    assert "l1.mlp.gate" not in shapes and "l1.norm2" not in shapes and shapes["l2.mlp.down"] == (72, 16)
    with pytest.raises(ValueError):
        gitopel.config_from_dict(dict(cfgd, layers=[{"type": "conv", "mixer": {}, "mlp": None}]))


def test_paged_cache_bookkeeping():
    from umbrella_amd.attn.cache import PagedSeqCache
    c = PagedSeqCache([(2, 8, 3)], [(1, 4, 4)], max_tokens=20, max_seqs=3, device="cpu", dtype=torch.bfloat16, page=4)
    assert c.n_pages == 8 and c.kv[0]["kp"].shape == (8, 2, 2, 8) and c.state[0].shape == (3, 1, 4, 4)
    assert c.open("a") == 0 and c.open("b") == 1
    assert c.extend("a", 5) == 0 and c.extend("a", 3) == 5 and c.length("a") == 8
    assert c.seqs["a"]["pages"] == [0, 1] and c.pages_dev[0, :2].tolist() == [0, 1]
    assert c.extend("b", 9) == 0 and c.seqs["b"]["pages"] == [2, 3, 4]
    assert c.extend("a", 1) == 8 and c.seqs["a"]["pages"] == [0, 1, 5]
    assert not c.can_extend("b", 12) and c.can_extend("b", 11)
    with pytest.raises(RuntimeError):
        c.extend("b", 12)
    assert c.length("b") == 9                                  # a refused extension changes nothing
    c.close("a")
    assert c.open("c") == 0                                    # the slot and the pages given back last go out first
    c.extend("c", 6)
    assert c.seqs["c"]["pages"] == [0, 1]
    with pytest.raises(KeyError):
        c.open("c")
    assert c.tokens_held() == 15
    c.clear()
    assert not c.seqs and len(c.free_pages) == 8 and len(c.free_slots) == 3


def test_oracle_visibility_rules():
    from oracle import seqmix as O
    assert O.visible_tokens(0, 4) == [0] and O.visible_tokens(10, 4) == [7, 8, 9, 10] and O.visible_tokens(5, 1) == [5]
    # blocks of 3 behind a window of 4: block b is seen from position 3b + 2 + 4 on
    assert O.visible_blocks(5, 4, 3) == [] and O.visible_blocks(6, 4, 3) == [0] and O.visible_blocks(8, 4, 3) == [0]
    assert O.visible_blocks(9, 4, 3) == [0, 1]
    for i in range(40):                                        # a token is never seen twice, some are not seen at all
        toks, blks = O.visible_tokens(i, 5), O.visible_blocks(i, 5, 4)
        covered = [p for b in blks for p in range(4 * b, 4 * b + 4)]
        assert not set(toks) & set(covered) and max(covered, default=-1) < min(toks)


def test_oracle_gla_state_can_be_carried():
    from oracle import seqmix as O
    g = torch.Generator().manual_seed(0)
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)  # noqa: E731
    H, D, E, W, n = 2, 4, 3, 10, 9
    ws = (r(H * D, W), r(H * D, W), r(H * E, W), r(H * E, W), r(W, H * E), r(E), r(2, W), r(H * D, 2), r(H * D))
    X = r(n, W)
    whole, S = O.gated_linear_attention(X, *ws, H=H, D=D, E=E, tau=3.0, eps=1e-6)
    a, Sa = O.gated_linear_attention(X[:4], *ws, H=H, D=D, E=E, tau=3.0, eps=1e-6)
    b, Sb = O.gated_linear_attention(X[4:], *ws, H=H, D=D, E=E, tau=3.0, eps=1e-6, state=Sa)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-12) and torch.allclose(Sb, S, atol=1e-12)


class _StandInModel:
    """what the batch engine needs of a model: a paged cache and forward_batch; logits put all weight on (last token + 1)"""

    def __init__(self, vocab=50, slots=2, max_tokens=64, page=4):
        from types import SimpleNamespace
        from umbrella_amd.attn.cache import PagedSeqCache
        self.config = SimpleNamespace(vocab_size=vocab)
        self.kv_cache = PagedSeqCache([], [], max_tokens=max_tokens, max_seqs=slots, device="cpu", dtype=torch.float32, page=page)
        self.max_length, self.batch_size, self.eos_tokens, self.steps = 64, slots, [49], []

    def open(self, sid):
        return self.kv_cache.open(sid)

    def close(self, sid):
        self.kv_cache.close(sid)

    def clear(self):
        self.kv_cache.clear()

    def forward_batch(self, parts, want=None):
        self.steps.append([(sid, len(t)) for sid, t in parts])
        rows = []
        for (sid, t), w in zip(parts, want):
            self.kv_cache.extend(sid, len(t))
            for k in w:
                row = torch.zeros(self.config.vocab_size)
                row[(t[k] + 1) % self.config.vocab_size] = 1.0
                rows.append(row)
        return torch.stack(rows)


def test_batch_engine_scheduler_with_a_stand_in_model(monkeypatch):
    from umbrella_amd.speculation.auto_engine import AutoEngine
    from umbrella_amd.speculation.batch_engine import BatchEngine
    from umbrella_amd.speculation.speculation_utils import IdTokenizer
    monkeypatch.setattr(BatchEngine, "_sample", lambda self, logits, reqs: logits.argmax(-1).tolist())
    m = _StandInModel()
    e = AutoEngine.from_config("cpu", engine="batch", model="stand-in", target_model_obj=m, tokenizer=IdTokenizer())
    assert isinstance(e, BatchEngine)
    e.initialize()
    outs = e.generate_batch([[5, 6, 7], [20], [44, 45]], max_new_tokens=4)
    assert outs == [[8, 9, 10, 11], [21, 22, 23, 24], [46, 47, 48, 49]]
    # two slots: the first two requests are prefilled together and decoded together, the third waits for the batch to drain
    assert m.steps[0] == [(0, 3), (1, 1)] and m.steps[1:4] == [[(0, 1), (1, 1)]] * 3 and m.steps[4] == [(2, 2)]
    assert not m.kv_cache.seqs and len(m.kv_cache.free_pages) == m.kv_cache.n_pages
    # eos ends a request early and frees its slot while the other goes on
    m.steps.clear()
    outs = e.generate_batch([[47], [1]], max_new_tokens=5)
    assert outs == [[48, 49], [2, 3, 4, 5, 6]] and m.steps[2] == [(4, 1)]      # request ids go on counting: 3 and 4
    with pytest.raises(ValueError):
        e.submit(list(range(62)), max_new_tokens=8)
    with pytest.raises(AssertionError):
        AutoEngine.from_config("cpu", engine="static", model="x")          # speculation engines still need a draft


def test_seq_header_matches_the_bindings():
    import ctypes as C
    import __graft_entry__ as ge
    from umbrella_amd import _lib
    ge.build_seq()
    lib = _lib.load_seq()
    hdr = open(os.path.join(ROOT, "include", "umbrella_seq.h")).read()
    declared = set(re.findall(r"\b(umb_[a-z0-9_]+)\s*\(", hdr))
    assert declared == set(_lib.SEQ_SIGNATURES), declared ^ set(_lib.SEQ_SIGNATURES)
    for name in declared:
        assert hasattr(lib, name)
    assert lib.umb_seq_version().startswith(b"umbrella_seq")
    assert C.sizeof(_lib.UmbSeqLinear) == 24 and C.sizeof(_lib.UmbPagedKV) == 56
    base = 16 * 4 + 5 * 24 + 7 * 8 + 56 + 8 + 8 * 4 + 24 + 10 * 8 + 24 + 2 * 8 + 2 * 24
    # + activation / routing kinds and correction, stream tables, the distance-bias attention and state-space fields
    # + the retention / convolved-attention / matrix-memory fields, the capped activation's constants, the embedding flag
    assert C.sizeof(_lib.UmbSeqLayer) == base + (2 * 4 + 8) + 6 * 8 + (3 * 8 + 2 * 4 + 4 * 4) + (6 * 4 + 7 * 8) + \
        (8 + 4 * 4 + 2 * 8 + 4 * 4 + 2 * 8 + 4 * 4 + 2 * 4)
    assert C.sizeof(_lib.UmbSeqModel) == 32 + 16 + 24 + 8 + 16 + 8 and C.sizeof(_lib.UmbSeqWork) == 9 * 8 + 8 + 8 * 8 + 8 + 2 * 8
    assert C.sizeof(_lib.UmbSeqStep) == 16 + 9 * 8
