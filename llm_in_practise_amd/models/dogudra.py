"""Dogudra: a decoder-only hybrid of latent-attention and state-space layers with routed feed-forwards.

* embedding: the token row times a scale, plus a hashed row for the (previous, current) token pair;
* every layer is post-normed: ``x <- norm(alpha*x + mixer(x))``, then ``x <- norm(alpha*x + ff(x))`` — the sublayers
  read ``x`` itself, and norm weights are stored as offsets from one;
* ``latent_attention`` mixers: queries through a low-rank latent, keys and values as per-head up-projections of one
  small normed latent per token plus one rotated key part shared by the heads, a per-head sigmoid output gate; a layer
  may borrow the cached latents of an earlier layer (``kv_from``) and apply its own up-projections;
* ``mamba2`` mixers: a selective state space in its state-space-duality form (short causal convolution + SiLU on
  x|B|C, scalar decay per head, gate before a grouped RMS norm);
* feed-forwards: tanh-GELU MLPs, or a mixture of clipped-GLU experts routed by softmax scores with a selection-only
  correction, group-limited top-k, identity experts and an always-on shared expert.

Serving layout (MI355X): the residual stream, norms, softmax, router, step sizes, decays and recurrent state are
float; matrix products run in the activation dtype (bf16 with float accumulation, or float).  Per mixer, every
projection that reads the sublayer input is ONE GEMM whose column slices the kernels read in place.  The attention
cache holds only ``[latent | rotated key part]`` per token; the key up-projection is carried to the query side and
the value up-projection is applied after the weighted sum, so every head sweeps the same cache rows (prefill, chunks
and decode are the same kernels).  Tokens of a step are packed back to back (:class:`~.common.SeqBatch`), per-sequence
state lives in slots of a :class:`~.common.SeqStateCache` (latent rows, state-space matrices, convolution inputs and
the last token for the pair hash).

Checkpoint: ``config.json`` (``architecture: "Dogudra"``, ``vocab``, ``width``, ``layers`` [...], ``norm.eps``,
``postln_alpha``, ``embedding.scale``, ``embedding.bigram``) + ``model.safetensors`` with names ``embed``, ``bigram``,
``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``; linear weights ``[out, in]``.
"""
from __future__ import annotations

import copy
import dataclasses
import json
import math
import os

import torch
import torch.nn as nn

from ..ops import conv as C
from ..ops.activation import clipped_glu, gelu_tanh
from ..ops.attention import latent_attention, latent_kv_store, rotary_inv_freq
from ..ops.conv import short_conv
from ..ops.embedding import embed_pair
from ..ops.moe import moe_glu_experts, route_tokens
from ..ops.norm import gate_group_norm, rms_norm_act, rms_norm_f32, scaled_postnorm
from ..ops.recurrent import ssd_scan
from .common import SeqBatch, SeqStateCausalLM, SeqStateModel, _HeadWeight

MIXERS = ("latent_attention", "mamba2")
FEW_PAIRS = 64          # (token, expert) pairs up to which a prefill step streams experts pair by pair


@dataclasses.dataclass
class DogudraConfig:
    vocab: int
    width: int
    layers: list
    norm_eps: float = 1e-6
    postln_alpha: float = 1.0
    embedding_scale: float = 1.0
    bigram: dict | None = None               # {"buckets", "mul_prev", "mul_cur"}
    max_position_embeddings: int = 4096      # engine default only
    model_type: str = "dogudra"
    eos_token_id: int | None = None

    @classmethod
    def from_dict(cls, d: dict) -> "DogudraConfig":
        layers = copy.deepcopy(d["layers"])
        for i, lc in enumerate(layers):
            if lc["type"] not in MIXERS:
                raise ValueError(f"Dogudra: unknown layer type {lc['type']!r}")
            mlp = lc.get("mlp")
            if mlp is not None and mlp.get("kind", "dense") not in ("dense", "moe"):
                raise ValueError(f"Dogudra: unknown feed-forward kind {mlp.get('kind')!r}")
            src = lc["mixer"].get("kv_from") if lc["type"] == "latent_attention" else None
            if src is not None:
                ok = 0 <= int(src) < i and layers[int(src)]["type"] == "latent_attention" and \
                    layers[int(src)]["mixer"].get("kv_from") is None
                a, b = lc["mixer"], layers[int(src)]["mixer"] if ok else {}
                for k in ("kv_rank", "rot_dim", "rot"):       # what the cache fixes; a borrower may leave it out
                    a.setdefault(k, b.get(k))
                if not ok or any(a.get(k) != b.get(k) for k in ("kv_rank", "rot_dim", "rot")):
                    raise ValueError(f"Dogudra: layer {i} cannot take its latents from layer {src}")
        e = d.get("embedding", {})
        return cls(vocab=int(d["vocab"]), width=int(d["width"]), layers=layers,
                   norm_eps=float(d.get("norm", {}).get("eps", 1e-6)), postln_alpha=float(d.get("postln_alpha", 1.0)),
                   embedding_scale=float(e.get("scale", 1.0)), bigram=e.get("bigram"),
                   max_position_embeddings=int(d.get("max_position_embeddings", 4096)))

    @classmethod
    def from_pretrained(cls, path: str) -> "DogudraConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict:
        e = {"scale": self.embedding_scale}
        if self.bigram:
            e["bigram"] = self.bigram
        return {"architecture": "Dogudra", "vocab": self.vocab, "width": self.width, "layers": self.layers,
                "norm": {"eps": self.norm_eps}, "postln_alpha": self.postln_alpha, "embedding": e}

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


def tensor_shapes(cfg: DogudraConfig) -> dict[str, tuple]:
    """Every checkpoint tensor of a config and its shape (a size that only the checkpoint's tensors fix — the query
    rank, the number of taps — reads as 0 when the config leaves it out)."""
    Wd = cfg.width
    out = {"embed": (cfg.vocab, Wd), "final.norm": (Wd,), "head": (cfg.vocab, Wd)}
    if cfg.bigram:
        out["bigram"] = (int(cfg.bigram["buckets"]) + 1, Wd)
    for i, lc in enumerate(cfg.layers):
        p, m, q = f"l{i}.", lc["mixer"], f"l{i}.mix."
        out[p + "norm1"] = (Wd,)
        if lc["type"] == "latent_attention":
            H, dn, dr, dv, R, qr = (int(m.get(k, 0)) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            out.update({q + "dq": (qr, Wd), q + "dq.norm": (qr,), q + "uq": (H * (dn + dr), qr), q + "uk": (H * dn, R),
                        q + "uv": (H * dv, R), q + "g": (H, Wd), q + "o": (Wd, H * dv)})
            if m.get("kv_from") is None:
                out.update({q + "dkv": (R + dr, Wd), q + "dkv.norm": (R,)})
        else:
            H, P, N, G, taps = (int(m.get(k, 0)) for k in ("heads", "vdim", "state", "groups", "conv"))
            inner, ch = H * P, H * P + 2 * G * N
            out.update({q + "in": (inner + ch + H, Wd), q + "conv": (ch, taps), q + "conv.b": (ch,), q + "dt_bias": (H,),
                        q + "A_log": (H,), q + "D": (H,), q + "norm": (inner,), q + "o": (Wd, inner)})
        mlp = lc.get("mlp")
        if mlp is None:
            continue
        out[p + "norm2"] = (Wd,)
        q = p + "mlp."
        if mlp.get("kind", "dense") == "dense":
            out.update({q + "up": (int(mlp["ff"]), Wd), q + "down": (Wd, int(mlp["ff"]))})
        else:
            r, F = mlp["router"], int(mlp["expert"]["ff"])
            n = int(r["experts"]) + int(r.get("identity", 0))
            out.update({q + "router": (n, Wd), q + "correction": (n,)})
            for e in range(int(r["experts"])):
                out.update({f"{q}e{e}.gate": (F, Wd), f"{q}e{e}.up": (F, Wd), f"{q}e{e}.down": (Wd, F)})
            if mlp.get("shared"):
                Fs = int(mlp["shared"]["ff"])
                out.update({q + "shared.gate": (Fs, Wd), q + "shared.up": (Fs, Wd), q + "shared.down": (Wd, Fs)})
    return out


def random_weights(cfg: DogudraConfig, seed: int = 0) -> dict[str, torch.Tensor]:
    """Synthetic weights (benchmarks, smoke runs, tests): matrices ~ N(0, 1/in), norm offsets and corrections near 0,
    step-size biases and decay rates in a stable range."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith("conv"):
            t = torch.randn(shape, generator=g) * 0.4
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[1])
            if leaf in ("embed", "bigram"):
                t = t * math.sqrt(shape[1]) * 0.5
        elif name.endswith("dq.norm") or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            t = 1 + 0.1 * torch.randn(shape, generator=g)
        elif leaf == "dt_bias":
            t = torch.rand(shape, generator=g) * 3 - 3
        elif leaf == "A_log":
            t = torch.rand(shape, generator=g) * 2 - 1
        elif leaf == "D":
            t = 1 + 0.2 * torch.randn(shape, generator=g)
        elif leaf == "correction":
            t = 0.05 * torch.randn(shape, generator=g)
        else:                                   # norm offsets, conv bias
            t = 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(torch.bfloat16)
    return out


def _f32(t, dev):
    return t.to(device=dev, dtype=torch.float32).contiguous()


def _act(t, dtype, dev):
    return t.to(device=dev, dtype=dtype).contiguous()


def _chunk(n: int, cap: int = 128) -> tuple[int, int]:
    """``n`` channels as (count, width) with the largest width <= ``cap`` that divides ``n``."""
    w = min(n, cap)
    while n % w:
        w -= 1
    return n // w, w


class _Sublayer(nn.Module):
    """Holds tensors as buffers (``.to()`` moves them); names are python identifiers, not checkpoint names."""

    def put(self, name: str, t: torch.Tensor):
        self.register_buffer(name, t, persistent=False)


class LatentAttentionMixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.H, self.dn, self.dr, self.dv, self.R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        self.scale = float(m["scale"])
        rot = m.get("rot") or {}
        self.rot_dims = int(rot.get("dims", 0))
        self.kv_from = None if m.get("kv_from") is None else int(m["kv_from"])
        self.q_rank = W[p + "dq"].shape[0]
        parts = [W[p + "dq"]] + ([W[p + "dkv"]] if self.kv_from is None else []) + [W[p + "g"]]
        self.put("w_in", torch.cat([t.to(dtype) for t in parts], 0).to(dev).contiguous())
        self.put("q_norm", _f32(W[p + "dq.norm"], dev))
        if self.kv_from is None:
            self.put("kv_norm", _f32(W[p + "dkv.norm"], dev))
        self.put("w_uq", _act(W[p + "uq"], dtype, dev))
        self.put("w_uk", _act(W[p + "uk"], dtype, dev).view(self.H, self.dn, self.R))                  # [H, dn, R]
        self.put("w_uv", _act(W[p + "uv"].view(self.H, self.dv, self.R).transpose(1, 2), dtype, dev))  # [H, R, dv]
        self.put("w_o", _act(W[p + "o"], dtype, dev))
        self.put("inv_freq", rotary_inv_freq(self.rot_dims, float(rot.get("base", 10000.0))).to(dev))

    def state_spec(self) -> dict:
        return {"ckv": ((self.R + self.dr,), "kv")} if self.kv_from is None else {}

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        H, dn, dr, R, T = self.H, self.dn, self.dr, self.R, h.shape[0]
        P = h @ self.w_in.t()
        a = self.q_rank
        q = rms_norm_act(P[:, :a], self.q_norm, eps) @ self.w_uq.t()              # [T, H * (dn + dr)]
        if self.kv_from is None:
            ckv = st["ckv"]
            latent_kv_store(P[:, a:a + R + dr], self.kv_norm, self.inv_freq, ckv, self.rot_dims, eps, sb)
            a += R + dr
        else:
            ckv = sb.cache.layers[self.kv_from]["ckv"]
        q_abs = torch.bmm(q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1), self.w_uk)      # [H, T, R]
        oc = latent_attention(q_abs, q, ckv, P[:, a:a + H], self.inv_freq, H, dn, self.rot_dims, self.scale, sb,
                              sb.cache.decode_splits if sb.decode else 1)                   # [T, H, R], gated
        ov = torch.bmm(oc.transpose(0, 1), self.w_uv)                                        # [H, T, dv]
        return ov.transpose(0, 1).reshape(T, H * self.dv) @ self.w_o.t()


class Mamba2Mixer(_Sublayer):
    def __init__(self, m: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.H, self.P, self.N, self.G = (int(m[k]) for k in ("heads", "vdim", "state", "groups"))
        self.parts = int(m.get("norm_groups", 1))
        self.inner, self.ch = self.H * self.P, self.H * self.P + 2 * self.G * self.N
        if self.H % self.G or self.inner % self.parts:
            raise ValueError("Dogudra: heads must be a multiple of groups, the inner width of norm_groups")
        self.put("w_in", _act(W[p + "in"], dtype, dev))
        self.put("conv_w", _f32(W[p + "conv"], dev))
        self.put("conv_b", _f32(W[p + "conv.b"], dev))
        self.put("dt_bias", _f32(W[p + "dt_bias"], dev))
        self.put("a_log", _f32(W[p + "A_log"], dev))
        self.put("d_skip", _f32(W[p + "D"], dev))
        self.put("norm", _f32(W[p + "norm"], dev))
        self.put("w_o", _act(W[p + "o"], dtype, dev))
        gn = self.G * self.N
        (nx, wx), (nb, wb) = _chunk(self.inner), _chunk(gn)
        self.segs = [(0, nx, wx, C.SILU, None, 1.0), (self.inner, nb, wb, C.SILU, None, 1.0),
                     (self.inner + gn, nb, wb, C.SILU, None, 1.0)]

    def state_spec(self) -> dict:
        spec = {"S": ((self.H, self.P, self.N), "f32")}
        if self.conv_w.shape[1] > 1:
            spec["conv"] = ((self.conv_w.shape[1] - 1, self.ch), "act")
        return spec

    def forward(self, h, sb: SeqBatch, st: dict, eps: float):
        inner, gn = self.inner, self.G * self.N
        P = h @ self.w_in.t()                                   # [z | x | B | C | dt]
        xbc = short_conv(P[:, inner:inner + self.ch], self.conv_w, st.get("conv"), self.segs, sb, eps, bias=self.conv_b)
        y = ssd_scan(xbc[:, inner + gn:], xbc[:, inner:inner + gn], xbc[:, :inner], P[:, inner + self.ch:], self.dt_bias,
                     self.a_log, self.d_skip, st["S"], self.H, self.G, sb)
        return gate_group_norm(y, P[:, :inner], self.norm, self.parts, eps) @ self.w_o.t()


class DenseFF(_Sublayer):
    def __init__(self, mlp: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        self.put("w_up", _act(W[p + "up"], dtype, dev))
        self.put("w_down", _act(W[p + "down"], dtype, dev))

    def forward(self, h, sb: SeqBatch):
        return gelu_tanh(h @ self.w_up.t()) @ self.w_down.t()


class RoutedFF(_Sublayer):
    def __init__(self, mlp: dict, W: dict, p: str, dtype, dev):
        super().__init__()
        r = mlp["router"]
        self.E, self.top, self.scale = int(r["experts"]), int(r["top"]), float(r.get("scale", 1.0))
        gr = r.get("groups") or {}
        self.groups, self.keep = int(gr.get("count", 1)), int(gr.get("keep", gr.get("count", 1)))
        self.limit = float(mlp["expert"]["limit"])
        self.put("router", _f32(W[p + "router"], dev))
        self.put("correction", _f32(W[p + "correction"], dev) if p + "correction" in W else None)
        self.put("w_gu", torch.stack([torch.stack([W[f"{p}e{e}.gate"], W[f"{p}e{e}.up"]]) for e in range(self.E)])
                 .to(device=dev, dtype=dtype).contiguous())                                  # [E, 2, F, W]
        self.put("w_d", torch.stack([W[f"{p}e{e}.down"] for e in range(self.E)]).to(device=dev, dtype=dtype).contiguous())
        self.shared = mlp.get("shared") is not None
        if self.shared:
            self.shared_limit = float(mlp["shared"]["limit"])
            self.put("ws_gu", _act(torch.cat([W[p + "shared.gate"], W[p + "shared.up"]], 0), dtype, dev))
            self.put("ws_d", _act(W[p + "shared.down"], dtype, dev))

    def forward(self, h, sb: SeqBatch):
        idx, w = route_tokens(h, self.router, self.correction, self.top, self.groups, self.keep, self.scale)
        sh = clipped_glu(h @ self.ws_gu.t(), self.shared_limit) @ self.ws_d.t() if self.shared else None
        few = sb.decode or h.shape[0] * self.top <= FEW_PAIRS
        return moe_glu_experts(h, self.w_gu, self.w_d, idx, w, self.limit, sh, few)


class DogudraLayer(nn.Module):
    def __init__(self, cfg: DogudraConfig, i: int, W: dict, dtype, dev):
        super().__init__()
        lc, p = cfg.layers[i], f"l{i}."
        self.kind = lc["type"]
        mixer = LatentAttentionMixer if self.kind == "latent_attention" else Mamba2Mixer
        self.mix = mixer(lc["mixer"], W, p + "mix.", dtype, dev)
        t = _Sublayer()
        t.put("norm1", 1.0 + _f32(W[p + "norm1"], dev))            # stored as an offset from one
        mlp = lc.get("mlp")
        self.ff = None
        if mlp is not None:
            t.put("norm2", 1.0 + _f32(W[p + "norm2"], dev))
            self.ff = (DenseFF if mlp.get("kind", "dense") == "dense" else RoutedFF)(mlp, W, p + "mlp.", dtype, dev)
        self.t = t

    def forward(self, x, h, sb: SeqBatch, st: dict, eps: float, alpha: float, dtype):
        """``x`` float residual (updated in place), ``h`` its copy in the activation dtype; returns the new ``h``."""
        h = scaled_postnorm(x, self.mix(h, sb, st, eps), self.t.norm1, alpha, eps, dtype)
        if self.ff is not None:
            h = scaled_postnorm(x, self.ff(h, sb), self.t.norm2, alpha, eps, dtype)
        return h


class DogudraModel(SeqStateModel):
    split_keys = 32           # every head sweeps the same cache rows: decode wants many short key splits

    def __init__(self, cfg: DogudraConfig, W: dict, dtype, dev):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        self.embed_tokens = nn.Parameter(_act(W["embed"], dtype, dev), requires_grad=False)
        self.register_buffer("pair_table", _act(W["bigram"], dtype, dev) if cfg.bigram else None, persistent=False)
        if cfg.bigram and W["bigram"].shape[0] != int(cfg.bigram["buckets"]) + 1:
            raise ValueError("Dogudra: the pair table must have buckets + 1 rows")
        self.layers = nn.ModuleList([DogudraLayer(cfg, i, W, dtype, dev) for i in range(len(cfg.layers))])
        self.register_buffer("final_norm", 1.0 + _f32(W["final.norm"], dev), persistent=False)
        self.residual_tap = None          # a list: receives a copy of the float residual after every layer

    def state_specs(self) -> list[dict]:
        # after the layers' entries: the model's own (the last token of every sequence, for the pair hash)
        return [layer.mix.state_spec() for layer in self.layers] + [{"prev": ((), "i32")} if self.cfg.bigram else {}]

    def state_device(self):
        return self.embed_tokens.device

    def run(self, tokens: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
        """Packed tokens ``[T]`` through all layers; returns the final-normed hidden states ``[T, width]``."""
        cfg, bg = self.cfg, self.cfg.bigram or {}
        x, h = embed_pair(tokens, self.embed_tokens, self.pair_table, sb.cache.layers[-1].get("prev"),
                          cfg.embedding_scale, int(bg.get("mul_prev", 0)), int(bg.get("mul_cur", 0)), sb)
        for i, layer in enumerate(self.layers):
            h = layer(x, h, sb, sb.cache.layers[i], cfg.norm_eps, cfg.postln_alpha, self.dtype)
            if self.residual_tap is not None:
                self.residual_tap.append(x.clone())
        return rms_norm_f32(x, self.final_norm, cfg.norm_eps, self.dtype)


class DogudraForCausalLM(SeqStateCausalLM):
    """Dogudra on the shared sequence-state causal-LM frame (``models/common.py``)."""

    config_class = DogudraConfig

    def __init__(self, cfg: DogudraConfig, weights: dict[str, torch.Tensor], dtype=torch.bfloat16, device=None):
        super().__init__()
        dev = torch.device(device or "cpu")
        missing = [k for k in tensor_shapes(cfg) if k not in weights and not k.endswith("correction")]
        if missing:
            raise KeyError(f"Dogudra checkpoint lacks {missing[:6]}")
        self.config = cfg
        self.model = DogudraModel(cfg, weights, dtype, dev)
        self.lm_head = _HeadWeight(_act(weights["head"], dtype, dev))
        self.eval()

    @classmethod
    def from_config(cls, cfg: DogudraConfig, dtype=torch.bfloat16, device=None, seed: int = 0):
        return cls(cfg, random_weights(cfg, seed), dtype, device)
