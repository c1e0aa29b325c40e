"""Serving throughput of the Dogudra design (latent attention + state-space layers, routed feed-forwards) beside
Mobupel — the framework's other sequence-state hybrid — and Qwen3, all at equal width, layer count, vocabulary and
matrix parameter count (random weights, layer sizes of real models).

Same procedure as :mod:`.hybrid_serve` (whose ``measure`` runs here): the serving engine's own step functions,
prefill of ``batch`` prompts of ``prompt`` tokens packed in one step, then ``decode_steps`` decode steps for the whole
batch, eager and through the captured hipGraphs.  ``bench.py --workload dogudra-serve`` calls :func:`run`; the default
workload of ``bench.py`` is untouched.
"""
from __future__ import annotations

import torch

from .hybrid_serve import SIZES as HYBRID_SIZES, _params, measure, mobupel_config

SIZES = {
    # eight layers: own-cache attention, borrower, state space, borrower, twice; the first feed-forward is dense
    "w1024": dict(width=1024, heads=8, dim=64, rot=64, vdim=64, kv_rank=192, q_rank=384, sh=32, sp=64, sn=128, sg=2,
                  ff=2816, experts=8, identity=2, top=4, eff=512, groups=2, keep=1),
    "w2048": dict(width=2048, heads=16, dim=64, rot=64, vdim=64, kv_rank=192, q_rank=768, sh=64, sp=64, sn=128, sg=2,
                  ff=5632, experts=8, identity=2, top=4, eff=512, groups=2, keep=1),
}


def dogudra_config(s: dict, vocab: int = 32000) -> dict:
    def attn(kv_from=None):
        m = {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot"], "vdim": s["vdim"], "kv_rank": s["kv_rank"],
             "q_rank": s["q_rank"], "scale": (s["dim"] + s["rot"]) ** -0.5, "rot": {"base": 10000.0, "dims": s["rot"]}}
        if kv_from is not None:
            m["kv_from"] = kv_from
        return {"type": "latent_attention", "mixer": m}

    def ssm():
        return {"type": "mamba2", "mixer": {"heads": s["sh"], "vdim": s["sp"], "state": s["sn"], "groups": s["sg"],
                                            "conv": 4, "norm_groups": 1}}
    moe = {"kind": "moe", "expert": {"ff": s["eff"], "limit": 7.0}, "shared": {"ff": s["eff"], "limit": 7.0},
           "router": {"experts": s["experts"], "identity": s["identity"], "top": s["top"], "scale": 2.0,
                      "groups": {"count": s["groups"], "keep": s["keep"]}}}
    layers = [attn(), attn(0), ssm(), attn(0), attn(), attn(4), ssm(), attn(4)]
    for i, lc in enumerate(layers):
        lc["mlp"] = {"kind": "dense", "ff": s["ff"]} if i == 0 else moe
    return {"architecture": "Dogudra", "vocab": vocab, "width": s["width"], "layers": layers, "norm": {"eps": 1e-6},
            "postln_alpha": 1.0, "embedding": {"scale": 1.0, "bigram": {"buckets": 8191, "mul_prev": 131, "mul_cur": 5}}}


def build_trio(size: str, device, vocab: int = 32000):
    """(Dogudra, Mobupel, Qwen3): same width, 8 layers, same vocabulary; the feed-forward widths of the other two are
    chosen so that all three hold the same number of matrix parameters (within one feed-forward column)."""
    from ..models.dogudra import DogudraConfig, DogudraForCausalLM
    from ..models.mobupel import MobupelConfig, MobupelForCausalLM
    from ..models.qwen3 import Qwen3Config, Qwen3ForCausalLM
    s = SIZES[size]
    dog = DogudraForCausalLM.from_config(DogudraConfig.from_dict(dogudra_config(s, vocab)), torch.bfloat16, device)
    target, W, L = _params(dog), s["width"], 8
    hs = dict(HYBRID_SIZES[size])

    def mob_with(ff):
        hs["ff"] = ff
        return MobupelForCausalLM.from_config(MobupelConfig.from_dict(mobupel_config(hs, vocab)), torch.bfloat16, device,
                                              rank=64)
    p0 = _params(mob_with(64))
    per_col = hs["pairs"] * 2 * W                     # one more feed-forward column in every parallel layer
    mob = mob_with(max(64, int(64 + (target - p0) / per_col) // 64 * 64))
    attn = W * hs["lh"] * hs["ld"] * 2 + W * hs["lg"] * hs["ld"] * 2
    inter = max(256, int(((target - 2 * vocab * W) / L - attn) / (3 * W)) // 64 * 64)
    qcfg = Qwen3Config(vocab_size=vocab, hidden_size=W, intermediate_size=inter, num_hidden_layers=L,
                       num_attention_heads=hs["lh"], num_key_value_heads=hs["lg"], head_dim=hs["ld"],
                       max_position_embeddings=8192)
    qwen = Qwen3ForCausalLM.from_config(qcfg, dtype=torch.bfloat16, device=device).eval()
    qwen.requires_grad_(False)
    qwen.fuse_projections()
    return dog, mob, qwen


def run(sizes=("w1024", "w2048"), batch: int = 8, prompt: int = 1024, decode_steps: int = 32, vocab: int = 32000,
        device=None, models=("dogudra", "mobupel", "qwen3"), graphs=(False, True)) -> dict:
    dev = torch.device(device or "cuda")
    out = {"metric": "dogudra_serve_tokens_per_s", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
           "batch": batch, "prompt": prompt, "decode_steps": decode_steps, "results": []}
    for size in sizes:
        trio = dict(zip(("dogudra", "mobupel", "qwen3"), build_trio(size, dev, vocab)))
        rec = {"size": size, **{f"{k}_params_m": round(_params(m) / 1e6, 1) for k, m in trio.items()}}
        for name in models:
            for g in graphs:
                rec[f"{name}_{'graphs' if g else 'eager'}"] = measure(trio[name], batch, prompt, decode_steps, g, vocab)
        out["results"].append(rec)
        del trio
        torch.cuda.empty_cache()
    return out
