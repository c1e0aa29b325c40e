"""Serving throughput of the hybrid recurrent / attention design (Mobupel) beside Qwen3 at equal size.

Both models run through the serving engine's step functions (``ServingEngine.forward_prefill`` /
``forward_decode``) with random weights at layer sizes of real models: prefill of ``batch`` prompts of ``prompt``
tokens packed in one step, then ``decode_steps`` decode steps for the whole batch (eager, and through the captured
hipGraphs).  Printed: tokens/s for both phases, both models, and their parameter counts.  ``bench.py --workload
hybrid-serve`` calls :func:`run`; the default workload of ``bench.py`` is untouched.
"""
from __future__ import annotations

import queue
import time

import torch

SIZES = {
    # width, layer pairs (one mlstm + one parallel layer each), heads
    "w1024": dict(width=1024, pairs=4, mh=8, mdk=64, mdv=96, lh=8, lg=2, ld=128, rh=4, rg=2, rd=128, ff=2048),
    "w2048": dict(width=2048, pairs=4, mh=8, mdk=128, mdv=192, lh=16, lg=4, ld=128, rh=8, rg=4, rd=128, ff=4096),
}


def mobupel_config(s: dict, vocab: int = 32000) -> dict:
    layers = []
    for _ in range(s["pairs"]):
        layers.append({"type": "mlstm", "mlp": None,
                       "mixer": {"heads": s["mh"], "dim": s["mdk"], "vdim": s["mdv"], "gate_cap": 15.0}})
        layers.append({"type": "parallel", "mlp": {"kind": "dense", "ff": s["ff"]},
                       "mixer": {"left": {"heads": s["lh"], "kv_heads": s["lg"], "dim": s["ld"], "vdim": s["ld"],
                                          "conv": 4, "scale": s["ld"] ** -0.5},
                                 "right": {"heads": s["rh"], "kv_heads": s["rg"], "dim": s["rd"], "vdim": s["rd"],
                                           "conv": 4}}})
    return {"architecture": "Mobupel", "vocab": vocab, "width": s["width"], "layers": layers, "norm": {"eps": 1e-6},
            "embedding": {"scale": 1.0}, "logit_scale": 1.0}


def _params(m) -> int:
    seen, n = set(), 0
    for t in list(m.parameters()) + list(m.buffers()):
        if t.data_ptr() not in seen and t.dim() >= 2:
            seen.add(t.data_ptr())
            n += t.numel()
    return n


def build_pair(size: str, device, vocab: int = 32000):
    """(Mobupel, Qwen3) with the same width, layer count and vocabulary; Qwen3's feed-forward is sized so that the
    two hold the same number of matrix parameters (within one intermediate column)."""
    from ..models.mobupel import MobupelConfig, MobupelForCausalLM
    from ..models.qwen3 import Qwen3Config, Qwen3ForCausalLM
    s = SIZES[size]
    mob = MobupelForCausalLM.from_config(MobupelConfig.from_dict(mobupel_config(s, vocab)), torch.bfloat16, device, rank=64)
    L, W = 2 * s["pairs"], s["width"]
    attn = W * s["lh"] * s["ld"] * 2 + W * s["lg"] * s["ld"] * 2
    inter = max(256, int(((_params(mob) - 2 * vocab * W) / L - attn) / (3 * W)) // 64 * 64)
    qcfg = Qwen3Config(vocab_size=vocab, hidden_size=W, intermediate_size=inter, num_hidden_layers=L,
                       num_attention_heads=s["lh"], num_key_value_heads=s["lg"], head_dim=s["ld"],
                       max_position_embeddings=8192)
    qwen = Qwen3ForCausalLM.from_config(qcfg, dtype=torch.bfloat16, device=device).eval()
    qwen.requires_grad_(False)
    qwen.fuse_projections()
    return mob, qwen


@torch.no_grad()
def measure(lm, batch: int, prompt: int, decode_steps: int, graphs: bool, vocab: int, reps: int = 3) -> dict:
    from ..infer.engine import SamplingParams, ServingEngine, _Request
    dev = next(lm.parameters()).device
    eng = ServingEngine(lm, None, max_batch=batch, max_model_len=prompt + decode_steps * (reps + 1) + 8,
                        use_graphs=graphs, start=False)
    g = torch.Generator().manual_seed(0)

    def requests():
        return [(i, _Request(torch.randint(0, vocab, (prompt,), generator=g).tolist(), SamplingParams(), False,
                             queue.Queue(), time.time())) for i in range(batch)]

    def sync():
        torch.cuda.synchronize(dev)
    best_p = float("inf")
    for r in range(reps + 1):                      # first pass warms allocator, kernels and GEMM plans
        for i in range(batch):
            eng.release(i)
        new = requests()
        sync()
        t0 = time.perf_counter()
        h, pp = eng.forward_prefill(new)
        eng._head(h[pp.last])
        sync()
        if r:
            best_p = min(best_p, time.perf_counter() - t0)
    active = list(range(batch))
    eng.next_tok[:batch] = torch.randint(0, vocab, (batch,), generator=g).to(dev)
    best_d = float("inf")
    for r in range(reps + 1):
        sync()
        t0 = time.perf_counter()
        for _ in range(decode_steps):
            eng.forward_decode(active)
        sync()
        if r:
            best_d = min(best_d, time.perf_counter() - t0)
    return {"prefill_tok_s": round(batch * prompt / best_p), "prefill_ms": round(best_p * 1e3, 2),
            "decode_tok_s": round(batch * decode_steps / best_d), "decode_ms_per_step": round(best_d / decode_steps * 1e3, 3)}


def run(sizes=("w1024", "w2048"), batch: int = 8, prompt: int = 1024, decode_steps: int = 32, vocab: int = 32000,
        device=None) -> dict:
    dev = torch.device(device or "cuda")
    out = {"metric": "hybrid_serve_tokens_per_s", "unit": "tokens/s", "dtype": "bf16", "data": "synthetic",
           "batch": batch, "prompt": prompt, "decode_steps": decode_steps, "results": []}
    for size in sizes:
        mob, qwen = build_pair(size, dev, vocab)
        rec = {"size": size, "mobupel_params_m": round(_params(mob) / 1e6, 1), "qwen3_params_m": round(_params(qwen) / 1e6, 1)}
        for name, lm in (("mobupel", mob), ("qwen3", qwen)):
            for graphs in (False, True):
                rec[f"{name}_{'graphs' if graphs else 'eager'}"] = measure(lm, batch, prompt, decode_steps, graphs, vocab)
        out["results"].append(rec)
        del mob, qwen
        torch.cuda.empty_cache()
    return out
