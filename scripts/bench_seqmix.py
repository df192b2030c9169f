"""Prefill and decode throughput of the sequence-mixer family at layer sizes that resemble real models.  Random weights,
synthetic ids.

    python bench.py --family gitopel [--sizes 1b,8b] [--prompt-len 2048] [--decode-steps 64] [--batch 16]
        Gitopel beside the framework's Llama runtime at equal width / feed-forward / head sizes and layer count
    python bench.py --family fidizen [--sizes 1b,8b] ...
        Fidizen (latent attention, dense PolyNorm and routed-expert feed-forwards) beside Gitopel's windowed-attention
        layers -- the closest existing model: same runtime, cache manager and engine -- at equal width, heads, window,
        feed-forward width and layer count

    python bench.py --family tomopel [--sizes 1b,8b] ...
        Tomopel (two residual streams; softmax attention with a distance bias beside a state-space layer; minGRU layers; dense
        and routed relu^2 feed-forwards) beside Gitopel -- the closest existing model: grouped-query attention layers where
        Tomopel has its parallel mixer, gated-linear-attention layers (the same scan kernel) where it has a minGRU -- at
        equal width, heads x head size, feed-forward width and layer count

    python bench.py --family zusuvik [--sizes 1b,8b] ...
        Zusuvik (parallel blocks; retention layers; convolved capped attention beside a matrix memory; capped-GLU experts routed
        on the logits with a gated shared expert) beside Tomopel -- the closest existing model: its parallel mixer (attention
        beside a state-space layer on the same scans) where Zusuvik has its own, minGRU layers where it has retention, routed
        experts everywhere -- at equal width, heads x head size, state size, expert width and layer count

or directly: python scripts/bench_seqmix.py.  One JSON line: per size, ms and tokens/s of
  prefill   one prompt of --prompt-len tokens in one step (Llama: its chunked prompt path)
  decode    one token per step behind that prompt, batch 1 (both) and batch --batch (Gitopel; the Llama runtime is batch 1)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# width, ff, attention heads / kv heads / head size, GLA heads / key size / value size, window, pool, layers
SIZES = {
    "1b": dict(width=2048, ff=8192, heads=32, kv_heads=8, dim=64, gheads=8, gdim=128, gvdim=256, window=512, pool=16,
               pattern="aagaag", vocab=32000),
    "8b": dict(width=4096, ff=14336, heads=32, kv_heads=8, dim=128, gheads=16, gdim=128, gvdim=256, window=1024, pool=16,
               pattern="aag", vocab=32000),
}


# Fidizen: per head `dim` unrotated + `rot` rotated features, value size vdim, latents q_rank / kv_rank; layers alternate a
# dense feed-forward (width ff) and experts (each ff / 4 wide, two of eight used, plus a shared one: ff / 2 active per token)
FID_SIZES = {
    "1b": dict(width=2048, ff=8192, heads=16, dim=64, rot=32, vdim=64, q_rank=768, kv_rank=256, window=512, experts=8, top=2,
               layers=4, vocab=32000),
    "8b": dict(width=4096, ff=14336, heads=32, dim=128, rot=64, vdim=128, q_rank=1536, kv_rank=512, window=1024, experts=8,
               top=2, layers=2, vocab=32000),
}


# Tomopel: attention heads x dim (values vdim) over kv_heads, beside a state-space layer of s_heads x s_vdim with `state`
# features per head; "p" layers have the parallel mixer, "g" layers a minGRU of the model's width; feed-forwards alternate
# dense (ff) and experts (each ff / 4 wide, two of eight used, plus a shared one)
TOM_SIZES = {
    "1b": dict(width=2048, ff=8192, heads=32, kv_heads=8, dim=64, vdim=64, s_heads=32, s_vdim=64, state=128, groups=8, conv=4,
               experts=8, top=2, pattern="pgpp", vocab=32000, bias_rows=32, bias_max=2048),
    "8b": dict(width=4096, ff=14336, heads=32, kv_heads=8, dim=128, vdim=128, s_heads=64, s_vdim=64, state=128, groups=8, conv=4,
               experts=8, top=2, pattern="pg", vocab=32000, bias_rows=32, bias_max=2048),
}


# Zusuvik: "r" layers are retention (r_heads x r_dim keys, r_vdim values), "p" layers convolved attention (heads x dim over
# kv_heads, `conv` taps) beside a matrix memory (m_heads x m_dim keys, m_vdim values); every layer has experts (each ff / 4
# wide, two of eight used) and a shared one
ZUS_SIZES = {
    "1b": dict(width=2048, ff=8192, heads=32, kv_heads=8, dim=64, vdim=64, conv=4, m_heads=8, m_dim=128, m_vdim=256, r_heads=8,
               r_dim=128, r_vdim=256, experts=8, top=2, pattern="rprp", vocab=32000),
    "8b": dict(width=4096, ff=14336, heads=32, kv_heads=8, dim=128, vdim=128, conv=4, m_heads=16, m_dim=128, m_vdim=256, r_heads=16,
               r_dim=128, r_vdim=256, experts=8, top=2, pattern="rp", vocab=32000),
}


def zusuvik_config(s):
    layers = []
    mlp = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "expert": {"ff": s["ff"] // 4, "limit": 7.0},
           "shared": {"ff": s["ff"] // 4, "limit": 7.0}}
    for ch in s["pattern"]:
        if ch == "p":
            mixer = {"left": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["vdim"], "conv": s["conv"],
                              "rot": {"base": 500000.0, "dims": s["dim"], "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}},
                              "scale": s["dim"] ** -0.5, "softcap": 30.0},
                     "right": {"heads": s["m_heads"], "dim": s["m_dim"], "vdim": s["m_vdim"], "gate_cap": 15.0},
                     "left_scale": 1.0, "right_scale": 1.0}
            layers.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
        else:
            H = s["r_heads"]
            mixer = {"heads": H, "dim": s["r_dim"], "vdim": s["r_vdim"], "decay": [1.0 - 2.0 ** (-5 - 5 * h / max(H - 1, 1)) for h in range(H)],
                     "rot": {"base": 10000.0, "dims": s["r_dim"]}}
            layers.append({"type": "retention", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Zusuvik", "layers": layers, "norm": {"eps": 1e-6}, "vocab": s["vocab"], "width": s["width"], "logit_scale": 1.0}


def tomopel_config(s):
    layers = []
    for i, ch in enumerate(s["pattern"]):
        if ch == "p":
            mixer = {"left": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["vdim"],
                              "scale": s["dim"] ** -0.5, "bias_max": s["bias_max"], "q_temp": {"coef": 0.1, "every": 256}},
                     "right": {"heads": s["s_heads"], "vdim": s["s_vdim"], "state": s["state"], "groups": s["groups"],
                               "norm_groups": s["groups"], "conv": s["conv"]}, "left_scale": 1.0, "right_scale": 1.0}
            kind = "parallel"
        else:
            mixer, kind = {"width": s["width"]}, "mingru"
        if i % 2 == 0 and not s.get("all_moe"):
            mlp = {"kind": "dense", "ff": s["ff"]}
        else:
            mlp = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "expert": {"ff": s["ff"] // 4},
                   "shared": {"ff": s["ff"] // 4}}
        layers.append({"type": kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Tomopel", "layers": layers, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0}, "streams": 2,
            "residual_mult": 0.5, "vocab": s["vocab"], "width": s["width"]}


def fidizen_config(s):
    mixer = {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot"], "vdim": s["vdim"], "q_rank": s["q_rank"],
             "kv_rank": s["kv_rank"], "mask": {"size": s["window"]}, "rot": {"dims": s["rot"], "base": 10000.0},
             "scale": (s["dim"] + s["rot"]) ** -0.5}
    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            mlp = {"kind": "dense", "ff": s["ff"]}
        else:
            mlp = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "expert": {"ff": s["ff"] // 4},
                   "shared": {"ff": s["ff"] // 4}}
        layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    return {"architecture": "Fidizen", "layers": layers, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "embedding": {"scale": s["width"] ** 0.5}, "vocab": s["vocab"], "width": s["width"]}


def gitopel_config(s):
    layers = []
    for ch in s["pattern"]:
        if ch == "a":
            layers.append({"type": "attention", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"],
                           "vdim": s["dim"], "mask": {"size": s["window"], "pool": s["pool"]},
                           "rot": {"dims": s["dim"], "base": 10000.0}, "scale": s["dim"] ** -0.5},
                           "mlp": {"ff": s["ff"], "kind": "dense"}})
        else:
            layers.append({"type": "gla", "mixer": {"heads": s["gheads"], "dim": s["gdim"], "vdim": s["gvdim"], "tau": 16.0},
                           "mlp": {"ff": s["ff"], "kind": "dense"}})
    return {"architecture": "Gitopel", "layers": layers, "norm": {"eps": 1e-6, "groups": 4}, "vocab": s["vocab"], "width": s["width"]}


def device_state(cfg, dtype, seed=0, rank=16, shapes=None, zero_norms=False):
    """random checkpoint drawn on the device in the storage dtype"""
    from umbrella_amd.models import gitopel
    g = torch.Generator(device="cuda").manual_seed(seed)
    sd = {}
    for name, shape in (shapes or gitopel.tensor_shapes(cfg, rank)).items():
        leaf = name.split(".")[-1]
        if ".hc" in name:                               # stream tables near the plain residual
            base = torch.eye(shape[0]) if len(shape) == 2 else torch.full(shape, 1.0 if leaf == "out" else 1.0 / shape[0])
            sd[name] = (base.cuda() + 0.05 * torch.randn(shape, generator=g, device="cuda")).to(dtype)
        elif "norm" in leaf:
            sd[name] = torch.full(shape, 0.0 if zero_norms and "mix." not in name else 1.0, dtype=dtype, device="cuda")
        elif len(shape) == 1:
            sd[name] = (0.1 * torch.randn(shape, generator=g, device="cuda")).to(dtype)
        else:
            sd[name] = (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) / shape[1] ** 0.5).to(dtype)
    return sd


def timed(fn, reps):
    torch.cuda.synchronize()
    t0 = time.time()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.time() - t0) / reps * 1e3


def bench_gitopel(s, args, dtype, fidizen=False, tomopel=False, zusuvik=False):
    from umbrella_amd.models import fidizen as fid
    from umbrella_amd.models import gitopel
    from umbrella_amd.models import tomopel as tom
    from umbrella_amd.models import zusuvik as zus
    B, P, steps = args.batch, args.prompt_len, args.decode_steps
    kw = dict(batch_size=B + 1, max_length=P + 2 * steps + 8, max_tokens=(B + 1) * (P + 2 * steps + 8), device="cuda:0",
              dtype=dtype, max_step_tokens=max(P, B))
    if zusuvik:
        cfg = zus.config_from_dict(zusuvik_config(s))
        sd = device_state(cfg, dtype, shapes=zus.tensor_shapes(cfg), zero_norms=True)
        m = zus.Zusuvik("bench", state_dict=sd, config=cfg, **kw)
    elif tomopel:
        cfg = tom.config_from_dict(tomopel_config(s))
        sd = device_state(cfg, dtype, shapes=tom.tensor_shapes(cfg, s["bias_rows"]), zero_norms=True)
        m = tom.Tomopel("bench", state_dict=sd, config=cfg, **kw)
    elif fidizen:
        cfg = fid.config_from_dict(fidizen_config(s))
        m = fid.Fidizen("bench", state_dict=device_state(cfg, dtype, shapes=fid.tensor_shapes(cfg)), config=cfg, **kw)
    else:
        cfg = gitopel.config_from_dict(gitopel_config(s))
        m = gitopel.Gitopel("bench", state_dict=device_state(cfg, dtype), config=cfg, **kw)
    m.alloc()
    ids = torch.randint(0, s["vocab"], (P,), generator=torch.Generator().manual_seed(1)).tolist()
    out = {"weight_GB": round(m.weight_bytes() / 1e9, 3)}

    def prefill():
        m.open("p")
        m.forward_batch([("p", ids)])
        m.close("p")
    prefill()
    ms = timed(prefill, 3)
    out["prefill"] = {"tokens": P, "ms": round(ms, 3), "tokens_per_s": round(P / ms * 1e3)}
    for b in (1, B):
        seqs = [f"s{i}" for i in range(b)]
        for q in seqs:
            m.open(q)
        m.forward_batch([(q, ids) for q in seqs[:1]])
        for q in seqs[1:]:                              # the other contexts one by one (bounded workspace)
            m.forward_batch([(q, ids)])
        step = lambda: m.forward_batch([(q, [7]) for q in seqs])  # noqa: E731
        step()
        ms = timed(step, steps)
        out[f"decode_b{b}"] = {"context": P, "ms_per_step": round(ms, 4), "tokens_per_s": round(b / ms * 1e3),
                               "weight_stream_TBs": round(m.weight_bytes() / ms / 1e9, 3)}
        for q in seqs:
            m.close(q)
    return out


def bench_llama(s, args, dtype):
    os.environ.setdefault("UMBRELLA_SYNTHETIC", "1")
    from umbrella_amd.models.config import LlamaCfg
    from umbrella_amd.models.llama import Llama
    P, steps = args.prompt_len, args.decode_steps
    cfg = LlamaCfg(vocab_size=s["vocab"], hidden_size=s["width"], intermediate_size=s["ff"], num_hidden_layers=len(s["pattern"]),
                   num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"], head_dim=s["dim"], rope_scaling=None,
                   rope_theta=10000.0, eos_token_id=[], name="llama-equal-size")
    m = Llama("llama-equal-size", max_length=P + 2 * steps + 64, device="cuda:0", dtype=dtype, config=cfg)
    m.alloc()
    m.reserve(max(m.PREFILL_CHUNK, 64), logit_rows=64)
    ids = torch.randint(0, s["vocab"], (P,), dtype=torch.int32, generator=torch.Generator().manual_seed(1)).cuda()
    out = {"weight_GB": round(m.weight_bytes() / 1e9, 3)}
    m.prefill_tokens(ids, 0)
    ms = timed(lambda: m.prefill_tokens(ids, 0), 3)
    out["prefill"] = {"tokens": P, "ms": round(ms, 3), "tokens_per_s": round(P / ms * 1e3)}
    tok = torch.tensor([7], dtype=torch.int32, device="cuda")
    pos = torch.tensor([P], dtype=torch.int32, device="cuda")
    pre = torch.tensor([P], dtype=torch.int32, device="cuda")
    step = lambda: m.forward_explicit(tok, pos, pos, pre)  # noqa: E731
    step()
    ms = timed(step, steps)
    out["decode_b1"] = {"context": P, "ms_per_step": round(ms, 4), "tokens_per_s": round(1 / ms * 1e3),
                        "weight_stream_TBs": round(m.weight_bytes() / ms / 1e9, 3)}
    return out


def run_fidizen(args):
    """Fidizen beside Gitopel's windowed-attention layers at equal width, heads x head size, window, feed-forward width and
    layer count"""
    import __graft_entry__ as ge
    ge.build_seq()
    dtype = torch.bfloat16
    res = {}
    for name in args.sizes.split(","):
        s = FID_SIZES[name]
        res[name] = {"shape": dict(s)}
        res[name]["fidizen"] = bench_gitopel(s, args, dtype, fidizen=True)
        torch.cuda.empty_cache()
        if not args.no_gitopel:
            hd = s["dim"] + s["rot"]
            g = dict(width=s["width"], ff=s["ff"], heads=s["heads"], kv_heads=max(1, s["heads"] // 4), dim=hd, window=s["window"],
                     pool=16, pattern="a" * s["layers"], vocab=s["vocab"])
            res[name]["gitopel_attention_equal_size"] = bench_gitopel(g, args, dtype)
            torch.cuda.empty_cache()
    line = {"metric": "prefill / decode throughput, Fidizen beside Gitopel's attention layers at equal size", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic: random weights, random ids", "n_gpus": 1, "prompt_len": args.prompt_len,
            "decode_steps": args.decode_steps, "batch": args.batch, "sizes": res}
    print(json.dumps(line), flush=True)
    return line


def run_tomopel(args):
    """Tomopel beside Gitopel at equal width, heads x head size, feed-forward width and layer count: attention layers for the
    parallel mixers, gated-linear-attention layers for the minGRU layers"""
    import __graft_entry__ as ge
    ge.build_seq()
    dtype = torch.bfloat16
    res = {}
    for name in args.sizes.split(","):
        s = TOM_SIZES[name]
        res[name] = {"shape": dict(s)}
        res[name]["tomopel"] = bench_gitopel(s, args, dtype, tomopel=True)
        torch.cuda.empty_cache()
        if not args.no_gitopel:
            g = dict(width=s["width"], ff=s["ff"], heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], gheads=s["s_heads"] // 4,
                     gdim=s["state"], gvdim=4 * s["s_vdim"], window=args.prompt_len + 2 * args.decode_steps + 8, pool=16,
                     pattern=s["pattern"].replace("p", "a"), vocab=s["vocab"])
            res[name]["gitopel_equal_size"] = bench_gitopel(g, args, dtype)
            torch.cuda.empty_cache()
    line = {"metric": "prefill / decode throughput, Tomopel beside Gitopel at equal size", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic: random weights, random ids", "n_gpus": 1, "prompt_len": args.prompt_len,
            "decode_steps": args.decode_steps, "batch": args.batch, "sizes": res}
    print(json.dumps(line), flush=True)
    return line


def run_zusuvik(args):
    """Zusuvik beside Tomopel at equal width, heads x head size, state size, expert width and layer count: Tomopel's parallel
    mixer for Zusuvik's, minGRU layers for the retention layers, routed experts in every layer"""
    import __graft_entry__ as ge
    ge.build_seq()
    dtype = torch.bfloat16
    res = {}
    for name in args.sizes.split(","):
        s = ZUS_SIZES[name]
        res[name] = {"shape": dict(s)}
        res[name]["zusuvik"] = bench_gitopel(s, args, dtype, zusuvik=True)
        torch.cuda.empty_cache()
        if not args.no_gitopel:
            t = dict(width=s["width"], ff=s["ff"], heads=s["heads"], kv_heads=s["kv_heads"], dim=s["dim"], vdim=s["vdim"],
                     s_heads=s["m_heads"] * 4, s_vdim=s["m_vdim"] // 4, state=s["m_dim"], groups=8, conv=s["conv"], experts=s["experts"],
                     top=s["top"], pattern=s["pattern"].replace("r", "g"), vocab=s["vocab"], bias_rows=32, bias_max=2048, all_moe=True)
            res[name]["tomopel_equal_size"] = bench_gitopel(t, args, dtype, tomopel=True)
            torch.cuda.empty_cache()
    line = {"metric": "prefill / decode throughput, Zusuvik beside Tomopel at equal size", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic: random weights, random ids", "n_gpus": 1, "prompt_len": args.prompt_len,
            "decode_steps": args.decode_steps, "batch": args.batch, "sizes": res}
    print(json.dumps(line), flush=True)
    return line


def run(args):
    import __graft_entry__ as ge
    ge.build()
    dtype = torch.bfloat16
    res = {}
    for name in args.sizes.split(","):
        s = SIZES[name]
        res[name] = {"shape": {k: v for k, v in s.items()}}
        if not args.no_gitopel:
            res[name]["gitopel"] = bench_gitopel(s, args, dtype)
            torch.cuda.empty_cache()
        if not args.no_llama:
            res[name]["llama_equal_size"] = bench_llama(s, args, dtype)
            torch.cuda.empty_cache()
    line = {"metric": "prefill / decode throughput, sequence-mixer family beside Llama at equal size", "unit": "tokens/s",
            "dtype": "bf16", "data": "synthetic: random weights, random ids", "n_gpus": 1, "prompt_len": args.prompt_len,
            "decode_steps": args.decode_steps, "batch": args.batch, "sizes": res}
    print(json.dumps(line), flush=True)
    return line


def add_args(ap):
    ap.add_argument("--sizes", default="1b,8b")
    ap.add_argument("--decode-steps", type=int, default=64)
    ap.add_argument("--batch", type=int, default=16)
    ap.add_argument("--no-llama", action="store_true")
    ap.add_argument("--no-gitopel", action="store_true")


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--prompt-len", type=int, default=2048)
    ap.add_argument("--family", default="gitopel", choices=["gitopel", "fidizen", "tomopel", "zusuvik"])
    add_args(ap)
    a = ap.parse_args()
    {"fidizen": run_fidizen, "tomopel": run_tomopel, "zusuvik": run_zusuvik}.get(a.family, run)(a)
