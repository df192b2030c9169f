"""Host-side tests of the Zusuvik design: configuration reading, the unrolled loop, registry, checkpoint names, the rotary
frequency table, and the plain oracle against itself in portions (no GPU)."""
import json
import math
import os
import sys

import pytest
import torch

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(__file__))


def test_config_reading_unrolls_the_loop():
    from zusuvik_helpers import CONFIGS
    from umbrella_amd.models import zusuvik
    cfg = zusuvik.config_from_dict(CONFIGS["mixed"])
    # layers 1 .. 2 run three times: 0 | 1 2 | 1 2 | 1 2 | 3
    assert [ly.tensor_prefix for ly in cfg.layers] == ["l0.", "l1.", "l2.", "l1.", "l2.", "l1.", "l2.", "l3."]
    assert [ly.weights_of for ly in cfg.layers] == [None, None, None, 1, 2, 1, 2, None]
    assert [ly.add_embed for ly in cfg.layers] == [False, False, False, True, False, True, False, False]
    assert cfg.block == "parallel" and cfg.norm_offset == 1.0 and cfg.logit_scale == 1.5
    a = cfg.layers[1]
    assert a.mixer.kind == "attention_mlstm" and a.mixer.taps == 3 and a.mixer.softcap == 5.0 and a.mixer.m_pad == 8
    assert a.route == "top_logits" and a.act == "clamp_glu" and a.shared_gate and a.act_limit == 1.5 and a.shared_limit == 1.0
    assert cfg.layers[2].shared_ff == 0 and not cfg.layers[2].shared_gate and not cfg.layers[7].has_ff
    # no loop, a loop over everything, a loop of one pass
    assert [ly.weights_of for ly in zusuvik.config_from_dict(CONFIGS["plain"]).layers] == [None, None]
    assert [ly.add_embed for ly in zusuvik.config_from_dict(CONFIGS["odd"]).layers] == [False, False, True, False]
    once = dict(CONFIGS["plain"], loop={"start": 0, "stop": 2, "times": 1})
    assert len(zusuvik.config_from_dict(once).layers) == 2


def test_registry_resolves_the_architecture(tmp_path):
    from zusuvik_helpers import CONFIGS
    from umbrella_amd.models.auto_model import AutoModelLM
    from umbrella_amd.models.config import read_architecture
    from umbrella_amd.models.zusuvik import Zusuvik
    (tmp_path / "config.json").write_text(json.dumps(CONFIGS["odd"]))
    assert read_architecture(str(tmp_path)) == "Zusuvik"
    assert AutoModelLM._ARCHITECTURE_MAPPING["Zusuvik"] is Zusuvik
    m = AutoModelLM.from_pretrained(str(tmp_path), device="cpu")
    assert isinstance(m, Zusuvik) and len(m.config.layers) == 4


def test_synthetic_checkpoint_names_and_shapes():
    from zusuvik_helpers import CONFIGS, checkpoint
    cfg, sd = checkpoint(CONFIGS["mixed"])
    assert "head" not in sd and sd["embed"].shape == (90, 40)
    assert sd["l1.mix.left.q.conv"].shape == (32, 3) and sd["l1.mix.left.q.norm"].shape == (32,) and sd["l1.mix.right.norm"].shape == (21,)
    assert sd["l1.mlp.shared.sg"].shape == (1, 40) and "l2.mlp.shared.sg" not in sd and "l3.norm2" not in sd
    assert sd["l0.mix.g"].shape == (18, 40) and sd["l1.mix.right.i.b"].shape == (3,)


@pytest.mark.parametrize("scaling", [None, {"factor": 16.0, "low": 1.0, "high": 8.0, "original": 4096},
                                     {"factor": 3.0, "low": 2.0, "high": 5.0, "original": 100}])
def test_rotary_frequency_table_equals_the_scalar_statement(scaling):
    from oracle import zusuvik as O
    from umbrella_amd.models.config import rotary_frequencies
    for dims, base in ((24, 250000.0), (6, 50.0), (64, 10000.0)):
        rot = {"dims": dims, "base": base}
        if scaling:
            rot["scaling"] = scaling
        want = O.rotary_frequencies(rot)
        got = rotary_frequencies(base, dims, scaling)
        assert got.dtype == torch.float32 and float(((got.double() - want) / want).abs().max()) < 1e-7
    if scaling:                                           # all three branches are met
        f = 10000.0 ** (-2.0 * torch.arange(32, dtype=torch.float64) / 64)
        wl = 2 * math.pi / f
        o = scaling["original"]
        assert bool((wl < o / scaling["high"]).any()) and bool((wl > o / scaling["low"]).any())


@pytest.mark.parametrize("name", ["mixed", "odd", "plain"])
def test_oracle_in_portions_equals_whole(name):
    from oracle import zusuvik as O
    from zusuvik_helpers import CONFIGS, checkpoint
    cfgd = CONFIGS[name]
    _, sd = checkpoint(cfgd, seed=3)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfgd["vocab"], (23,), generator=g).tolist()
    whole, layers, _ = O.forward(cfgd, sd, toks)
    assert layers.shape[0] == len(O.layer_runs(cfgd))
    rows, st, at = [], None, 0
    for k in (5, 1, 1, 9, 2, 5):
        lg, _, st = O.forward(cfgd, sd, toks[at:at + k], st)
        rows.append(lg)
        at += k
    assert float((torch.cat(rows) - whole).abs().max()) < 1e-9
