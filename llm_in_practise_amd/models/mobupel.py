"""Mobupel: a decoder-only hybrid whose layers alternate two kinds of token mixer.

* ``mlstm`` layers: the matrix-memory cell of xLSTM (exponential input gate, sigmoid forget gate, both soft-capped,
  stabilised by a running maximum that starts at 0), read out through a per-head RMS norm and a sigmoid gate.
* ``parallel`` layers: two mixers read the same input and their RMS-normed outputs are averaged —
  ``left``: grouped-query softmax attention without positional rotation, whose q/k/v pass a short causal convolution,
  q/k a per-head RMS norm, and whose softmax weights are mixed across heads by a learned ``[H, H]`` matrix before they
  meet the values; ``right``: the gated delta rule (short convolutions + SiLU, unit-length q/k, a per-key-channel
  decay from a low-rank projection, write strength beta), read out like the mLSTM.
* every sublayer is ``x <- x + norm_b(sublayer(norm(x)) * sigmoid(W_rg norm(x) + b_rg))``; feed-forwards are
  ``down(PolyNorm(up h))``; positions enter once, as a sinusoidal vector added to the scaled embedding.

Serving layout (MI355X): the residual stream, norms, softmax, gates and recurrent state are float, matrix products
run in the activation dtype (bf16 with float accumulation, or float).  All projections that read a sublayer's input
are ONE GEMM (mixer projections | low-rank gate inputs | residual gate); the kernels read its column slices in place.
Tokens of a step are packed back to back (:class:`~.common.SeqBatch`), per-sequence state lives in slots of a
:class:`~.common.SeqStateCache`, so prefill, continued prefill, decode and mixed batches are the same code.  Per
layer: norm -> GEMM -> [conv+norm | scan | attention] kernels -> output GEMM -> fused gated-residual + next-norm.

Checkpoint: ``config.json`` (``architecture: "Mobupel"``, ``width``, ``vocab``, ``layers`` [...], ``norm.eps``,
``embedding.scale``, ``logit_scale``) + ``model.safetensors`` with names ``embed``, ``l<i>.norm1`` ...,
``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""
from __future__ import annotations

import dataclasses
import json
import math
import os

import torch
import torch.nn as nn

from ..ops import conv as C
from ..ops.activation import polynorm
from ..ops.attention import talking_heads_attention
from ..ops.conv import short_conv
from ..ops.embedding import embed_sincos, sinusoid_inv_freq
from ..ops.norm import dual_norm_mean, gated_residual_norm, head_norm_gate, rms_norm_f32
from ..ops.recurrent import decay_gate, gated_delta_scan, mlstm_scan
from .common import SeqBatch, SeqStateCausalLM, SeqStateModel, _HeadWeight


@dataclasses.dataclass
class MobupelConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    max_position_embeddings: int = 4096      # engine default only: sinusoidal positions have no trained limit
    model_type: str = "mobupel"
    eos_token_id: int | None = None

    @classmethod
    def from_dict(cls, d: dict) -> "MobupelConfig":
        for lc in d["layers"]:
            if lc["type"] not in ("mlstm", "parallel"):
                raise ValueError(f"Mobupel: unknown layer type {lc['type']!r}")
            if lc.get("mlp") is not None and lc["mlp"].get("kind", "dense") != "dense":
                raise ValueError(f"Mobupel: unknown feed-forward kind {lc['mlp'].get('kind')!r}")
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=d["layers"],
                   norm_eps=float(d.get("norm", {}).get("eps", 1e-6)),
                   embedding_scale=float(d.get("embedding", {}).get("scale", 1.0)),
                   logit_scale=float(d.get("logit_scale", 1.0)),
                   max_position_embeddings=int(d.get("max_position_embeddings", 4096)))

    @classmethod
    def from_pretrained(cls, path: str) -> "MobupelConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        return {"architecture": "Mobupel", "vocab": self.vocab, "width": self.width, "layers": self.layers,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "logit_scale": self.logit_scale}

    # names the serving engine and the CLI read from any causal-LM config
    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width


def tensor_shapes(cfg: MobupelConfig, rank: int = 16) -> dict[str, tuple]:
    """Every checkpoint tensor of a config and its shape (``rank``: the low-rank gates' inner size, which a
    checkpoint fixes by its own shapes)."""
    Wd, out = cfg.width, {"embed": (cfg.vocab, cfg.width), "final.norm": (cfg.width,), "head": (cfg.vocab, cfg.width)}
    for i, lc in enumerate(cfg.layers):
        p, m = f"l{i}.", lc["mixer"]
        out.update({p + "norm1": (Wd,), p + "norm1b": (Wd,), p + "rg1": (Wd, Wd), p + "rg1.b": (Wd,)})
        if lc["type"] == "mlstm":
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            q = p + "mix."
            out.update({q + "q": (H * dk, Wd), q + "k": (H * dk, Wd), q + "v": (H * dv, Wd), q + "g": (H * dv, Wd),
                        q + "o": (Wd, H * dv), q + "norm": (H * dv,), q + "i": (H, Wd), q + "i.b": (H,),
                        q + "f": (H, Wd), q + "f.b": (H,)})
        else:
            l, r = m["left"], m["right"]
            q = p + "mix.left."
            H, G, dk, dv = l["heads"], l["kv_heads"], l["dim"], l["vdim"]
            out.update({q + "q": (H * dk, Wd), q + "k": (G * dk, Wd), q + "v": (G * dv, Wd), q + "q.norm": (dk,),
                        q + "k.norm": (dk,), q + "talk": (H, H), q + "g": (H * dv, Wd), q + "o": (Wd, H * dv)})
            if l.get("conv"):
                out.update({q + "q.conv": (H * dk, l["conv"]), q + "k.conv": (G * dk, l["conv"]),
                            q + "v.conv": (G * dv, l["conv"])})
            q = p + "mix.right."
            H, G, dk, dv, taps = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            out.update({q + "q": (G * dk, Wd), q + "k": (G * dk, Wd), q + "v": (H * dv, Wd), q + "q.conv": (G * dk, taps),
                        q + "k.conv": (G * dk, taps), q + "v.conv": (H * dv, taps), q + "b": (H, Wd), q + "A_log": (H,),
                        q + "norm": (dv,), q + "a1": (rank, Wd), q + "a2": (H * dk, rank), q + "dt_bias": (H * dk,),
                        q + "g1": (rank, Wd), q + "g2": (H * dv, rank), q + "o": (Wd, H * dv),
                        p + "mix.left.out": (Wd,), p + "mix.right.out": (Wd,)})
        if lc.get("mlp") is not None:
            ff = lc["mlp"]["ff"]
            out.update({p + "norm2": (Wd,), p + "norm2b": (Wd,), p + "rg2": (Wd, Wd), p + "rg2.b": (Wd,),
                        p + "mlp.up": (ff, Wd), p + "mlp.down": (Wd, ff), p + "mlp.act": (4,)})
    return out


def random_weights(cfg: MobupelConfig, seed: int = 0, rank: int = 16) -> dict[str, torch.Tensor]:
    """Synthetic weights (benchmarks, smoke runs): matrices ~ N(0, 1/in), norm weights near 1, gate biases that keep
    the recurrences in a stable range."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg, rank).items():
        leaf = name.rsplit(".", 1)[-1]
        if len(shape) == 2 and leaf not in ("conv", "talk"):
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.4
        elif leaf == "talk":
            t = torch.eye(shape[0]) + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "act":
            t = torch.tensor([0.7, 0.3, 0.15, 0.05])
        elif name.endswith("f.b"):
            t = torch.rand(shape, generator=g) * 3 + 1
        elif leaf in ("A_log", "dt_bias"):
            t = -torch.rand(shape, generator=g) * 3
        elif leaf == "b":
            t = torch.randn(shape, generator=g) * 0.1
        else:
            t = 1 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16)
    return out


def _f32(t, dev):
    return t.to(device=dev, dtype=torch.float32).contiguous()


class _Sublayer(nn.Module):
    """Holds tensors as buffers (``.to()`` moves them); names are python identifiers, not checkpoint names."""

    def put(self, name: str, t: torch.Tensor):
        self.register_buffer(name, t, persistent=False)


class MlstmMixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev, extra_in: list):
        super().__init__()
        self.H, self.dk, self.dv, self.cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
        parts = [W[p + "q"], W[p + "k"], W[p + "v"], W[p + "g"]] + extra_in
        self.put("w_in", torch.cat([t.to(dtype) for t in parts], 0).to(dev).contiguous())
        self.put("w_gate", _f32(torch.cat([W[p + "i"], W[p + "f"]], 0), dev))
        self.put("ib", _f32(W[p + "i.b"], dev))
        self.put("fb", _f32(W[p + "f.b"], dev))
        self.put("norm", _f32(W[p + "norm"], dev))
        self.put("w_o", W[p + "o"].to(device=dev, dtype=dtype).contiguous())
        self.n_in = sum(t.shape[0] for t in parts[:4])

    def state_spec(self) -> dict:
        return {"S": ((self.H, self.dv, self.dk), "f32"), "n": ((self.H, self.dk), "f32"), "m": ((self.H,), "f32")}

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        H, dk, dv = self.H, self.dk, self.dv
        P = h @ self.w_in.t()
        gates = h.float() @ self.w_gate.t()
        a, b = H * dk, 2 * H * dk
        o, den, floor = mlstm_scan(P[:, :a], P[:, a:b], P[:, b:b + H * dv], gates[:, :H].contiguous(),
                                   gates[:, H:].contiguous(), self.ib, self.fb, self.cap, dk ** -0.5, st["S"], st["n"],
                                   st["m"], H, sb)
        y = head_norm_gate(o, self.norm, P[:, b + H * dv:b + 2 * H * dv], eps, den, floor)
        return y @ self.w_o.t(), P[:, self.n_in:]


class ParallelMixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev, extra_in: list):
        super().__init__()
        l, r = m["left"], m["right"]
        self.LH, self.LG, self.Ldk, self.Ldv = int(l["heads"]), int(l["kv_heads"]), int(l["dim"]), int(l["vdim"])
        self.scale = float(l["scale"])
        self.RH, self.RG, self.Rdk, self.Rdv = int(r["heads"]), int(r["kv_heads"]), int(r["dim"]), int(r["vdim"])
        if self.LH % self.LG or self.RH % self.RG:
            raise ValueError("Mobupel: heads must be a multiple of kv_heads")
        L, R = p + "left.", p + "right."
        self.rank_g = W[R + "g1"].shape[0]
        parts = [W[L + "q"], W[L + "k"], W[L + "v"], W[L + "g"], W[R + "q"], W[R + "k"], W[R + "v"], W[R + "g1"]]
        self.put("w_in", torch.cat([t.to(dtype) for t in parts + extra_in], 0).to(dev).contiguous())
        self.n_in = sum(t.shape[0] for t in parts)
        self.CL = (self.LH + self.LG) * self.Ldk + self.LG * self.Ldv
        self.CR = 2 * self.RG * self.Rdk + self.RH * self.Rdv

        def conv_w(prefix, names, widths):      # a mixer without the tensors has no convolution: one tap of 1
            if prefix + names[0] + ".conv" in W:
                return _f32(torch.cat([W[prefix + n + ".conv"] for n in names], 0), dev)
            return torch.ones(sum(widths), 1, dtype=torch.float32, device=dev)
        self.put("conv_l", conv_w(L, "qkv", [self.LH * self.Ldk, self.LG * self.Ldk, self.LG * self.Ldv]))
        self.put("conv_r", conv_w(R, "qkv", [self.RG * self.Rdk, self.RG * self.Rdk, self.RH * self.Rdv]))
        self.put("qn", _f32(W[L + "q.norm"], dev))
        self.put("kn", _f32(W[L + "k.norm"], dev))
        self.put("talk", _f32(W[L + "talk"], dev))
        self.put("w_ol", W[L + "o"].to(device=dev, dtype=dtype).contiguous())
        self.put("w_small", _f32(torch.cat([W[R + "b"], W[R + "a1"]], 0), dev))
        self.put("w_a2", _f32(W[R + "a2"], dev))
        self.put("dt_bias", _f32(W[R + "dt_bias"], dev))
        self.put("a_log", _f32(W[R + "A_log"], dev))
        self.put("w_g2", W[R + "g2"].to(device=dev, dtype=dtype).contiguous())
        self.put("rnorm", _f32(W[R + "norm"], dev))
        self.put("w_or", W[R + "o"].to(device=dev, dtype=dtype).contiguous())
        self.put("out_l", _f32(W[p + "left.out"], dev))
        self.put("out_r", _f32(W[p + "right.out"], dev))

    def state_spec(self) -> dict:
        spec = {"k": ((self.LG * self.Ldk,), "kv"), "v": ((self.LG * self.Ldv,), "kv"),
                "S": ((self.RH, self.Rdv, self.Rdk), "f32")}
        if self.conv_l.shape[1] > 1:
            spec["lconv"] = ((self.conv_l.shape[1] - 1, self.CL), "act")
        if self.conv_r.shape[1] > 1:
            spec["rconv"] = ((self.conv_r.shape[1] - 1, self.CR), "act")
        return spec

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        H, G, dk, dv = self.LH, self.LG, self.Ldk, self.Ldv
        P = h @ self.w_in.t()
        # ---- left: convolved, normed q/k -> cache -> attention with head-mixed weights
        nq, nk, nv = H * dk, G * dk, G * dv
        cl = short_conv(P[:, :self.CL], self.conv_l, st.get("lconv"),
                        [(0, H, dk, C.RMS, self.qn, 1.0), (nq, G, dk, C.RMS, self.kn, 1.0), (nq + nk, G, dv, C.PLAIN, None, 1.0)],
                        sb, eps)
        st["k"].view(-1, nk).index_copy_(0, sb.cache_idx, cl[:, nq:nq + nk])
        st["v"].view(-1, nv).index_copy_(0, sb.cache_idx, cl[:, nq + nk:])
        c0 = self.CL
        ol = talking_heads_attention(cl[:, :nq], st["k"], st["v"], self.talk, P[:, c0:c0 + H * dv], H, G, self.scale, sb,
                                     sb.cache.decode_splits if sb.decode else 1)
        yl = ol @ self.w_ol.t()
        # ---- right: gated delta rule
        c0 += H * dv
        H, G, dk, dv = self.RH, self.RG, self.Rdk, self.Rdv
        cr = short_conv(P[:, c0:c0 + self.CR], self.conv_r, st.get("rconv"),
                        [(0, G, dk, C.SILU_UNIT, None, dk ** -0.5), (G * dk, G, dk, C.SILU_UNIT, None, 1.0),
                         (2 * G * dk, H, dv, C.SILU, None, 1.0)], sb, eps, out_f32=True)
        small = h.float() @ self.w_small.t()
        g = decay_gate(small[:, H:] @ self.w_a2.t(), self.dt_bias, self.a_log, dk)
        o = gated_delta_scan(cr[:, :G * dk], cr[:, G * dk:2 * G * dk], cr[:, 2 * G * dk:], g, small[:, :H].contiguous(),
                             st["S"], H, G, sb)
        c0 += self.CR
        gate2 = P[:, c0:c0 + self.rank_g] @ self.w_g2.t()
        yr = head_norm_gate(o, self.rnorm, gate2, eps) @ self.w_or.t()
        return dual_norm_mean(yl, yr, self.out_l, self.out_r, eps), P[:, self.n_in:]


class MobupelLayer(nn.Module):
    def __init__(self, cfg: MobupelConfig, i: int, W: dict, dtype, dev):
        super().__init__()
        lc, p = cfg.layers[i], f"l{i}."
        self.kind = lc["type"]
        mixer = MlstmMixer if self.kind == "mlstm" else ParallelMixer
        self.mix = mixer(lc["mixer"], W, p + "mix.", dtype, dev, [W[p + "rg1"]])
        t = _Sublayer()
        for name in ("norm1", "norm1b", "rg1.b"):
            t.put(name.replace(".", "_"), _f32(W[p + name], dev))
        self.has_mlp = lc.get("mlp") is not None
        if self.has_mlp:
            for name in ("norm2", "norm2b", "rg2.b", "mlp.act"):
                t.put(name.replace(".", "_"), _f32(W[p + name], dev))
            for name in ("mlp.up", "mlp.down", "rg2"):
                t.put(name.replace(".", "_"), W[p + name].to(device=dev, dtype=dtype).contiguous())
        self.t = t

    def forward(self, x, h, sb: SeqBatch, st: dict, eps: float, next_norm):
        """``x`` float residual (updated in place), ``h = norm1(x)``; returns the next layer's normed input."""
        t = self.t
        y, rg = self.mix(h, sb, st, eps)
        h = gated_residual_norm(x, y, rg, t.rg1_b, t.norm1b, t.norm2 if self.has_mlp else next_norm, eps)
        if self.has_mlp:
            y = polynorm(h @ t.mlp_up.t(), t.mlp_act, eps) @ t.mlp_down.t()
            h = gated_residual_norm(x, y, h @ t.rg2.t(), t.rg2_b, t.norm2b, next_norm, eps)
        return h


class MobupelModel(SeqStateModel):
    def __init__(self, cfg: MobupelConfig, W: dict, dtype, dev):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.embed_tokens = nn.Parameter(W["embed"].to(device=dev, dtype=dtype).contiguous(), requires_grad=False)
        self.register_buffer("inv_freq", sinusoid_inv_freq(cfg.width).to(dev), persistent=False)
        self.layers = nn.ModuleList([MobupelLayer(cfg, i, W, dtype, dev) for i in range(len(cfg.layers))])
        self.register_buffer("final_norm", _f32(W["final.norm"], dev), persistent=False)
        self.residual_tap = None          # a list: receives a copy of the float residual after every layer

    def state_specs(self) -> list[dict]:
        return [layer.mix.state_spec() for layer in self.layers]

    def state_device(self):
        return self.embed_tokens.device

    def run(self, tokens: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
        """Packed tokens ``[T]`` through all layers; returns the final-normed hidden states ``[T, width]``."""
        eps, L = self.cfg.norm_eps, self.layers
        x = embed_sincos(tokens, sb.desc[4], self.embed_tokens, self.inv_freq, self.cfg.embedding_scale)
        h = rms_norm_f32(x, L[0].t.norm1, eps, self.dtype)
        for i, layer in enumerate(L):
            nxt = L[i + 1].t.norm1 if i + 1 < len(L) else self.final_norm
            h = layer(x, h, sb, sb.cache.layers[i], eps, nxt)
            if self.residual_tap is not None:
                self.residual_tap.append(x.clone())
        return h


class MobupelForCausalLM(SeqStateCausalLM):
    """Mobupel on the shared sequence-state causal-LM frame (``models/common.py``)."""

    config_class = MobupelConfig

    def __init__(self, cfg: MobupelConfig, weights: dict[str, torch.Tensor], dtype=torch.bfloat16, device=None):
        super().__init__()
        dev = torch.device(device or "cpu")
        missing = [k for k in tensor_shapes(cfg, 1) if k not in weights]
        if missing:
            raise KeyError(f"Mobupel checkpoint lacks {missing[:6]}")
        self.config = cfg
        self.model = MobupelModel(cfg, weights, dtype, dev)
        self.lm_head = _HeadWeight(weights["head"].to(device=dev, dtype=dtype).contiguous())
        self.logit_scale = cfg.logit_scale
        self.eval()

    @classmethod
    def from_config(cls, cfg: MobupelConfig, dtype=torch.bfloat16, device=None, seed: int = 0, rank: int = 16):
        return cls(cfg, random_weights(cfg, seed, rank), dtype, device)
