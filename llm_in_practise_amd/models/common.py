"""Shared model plumbing: fused projections, output container, KV cache."""
from __future__ import annotations

import dataclasses

import torch
import torch.nn as nn

from ..ops.linear import LoraBranch, fused_linear
from ..peft.lora import Linear4bit, LoraLayer, base_of
from ..quant.int4 import Int4Linear, Int4Weight, int4_linear
from ..quant.nf4 import NF4Weight, concat_nf4


@dataclasses.dataclass
class CausalLMOutput:
    loss: torch.Tensor | None = None
    logits: torch.Tensor | None = None
    past_key_values: object | None = None
    hidden_states: torch.Tensor | None = None

    def __getitem__(self, i):
        return [v for v in (self.loss, self.logits) if v is not None][i]


def _leaf_linear(m: nn.Module) -> nn.Module:
    return m.base_layer if isinstance(m, LoraLayer) else m


def _out_features(m: nn.Module) -> int:
    return _leaf_linear(m).out_features


def _trainable_base(m: nn.Module) -> bool:
    leaf = _leaf_linear(m)
    return isinstance(leaf, nn.Linear) and leaf.weight.requires_grad


class FusedProjection:
    """Row-concatenation of projections that share one input (q|k|v, gate|up).

    The concatenated base replaces the parts' storage (each part's buffers / weight become
    views into it), so fusion costs no extra HBM.  LoRA branches keep their own A/B and
    address their column range of the fused output.  Not used when a base weight is
    trainable (full fine-tune) — then each projection runs on its own.
    """

    def __init__(self, mods: list[nn.Module]):
        self.mods = mods
        leaves = [_leaf_linear(m) for m in mods]
        self.splits = [_out_features(m) for m in mods]
        if all(isinstance(l, Linear4bit) for l in leaves):
            parts = [l.nf4 for l in leaves]
            fused = concat_nf4(parts)
            self.base: NF4Weight | torch.Tensor = fused
            r0, b0 = 0, 0
            for l in leaves:                      # re-point parts at views of the fused storage
                n = l.out_features
                nblk = n * l.in_features // l.blocksize
                l.codes = fused.codes[r0:r0 + n]
                if fused.double_quant:
                    g0, ng = b0 // 256, nblk // 256
                    l.qabsmax = fused.qabsmax[b0:b0 + nblk]
                    l.absmax2 = fused.absmax2[g0:g0 + ng]
                    l.offset = fused.offset[g0:g0 + ng]
                else:
                    l.absmax = fused.absmax[b0:b0 + nblk]
                r0 += n
                b0 += nblk
            biases = [l.bias for l in leaves]
        elif all(isinstance(l, Int4Linear) for l in leaves):   # W4A16 (GPTQ / AWQ / RTN): concat along N
            codes = torch.cat([l.codes for l in leaves], 0)
            scales = torch.cat([l.scales for l in leaves], 0)
            zeros = torch.cat([l.zeros for l in leaves], 0)
            self.base = Int4Weight(codes, scales, zeros, (codes.shape[0], leaves[0].in_features),
                                   leaves[0].group_size, leaves[0].sym)
            r0 = 0
            for l in leaves:
                n = l.out_features
                l.load(Int4Weight(codes[r0:r0 + n], scales[r0:r0 + n], zeros[r0:r0 + n], (n, l.in_features),
                                  l.group_size, l.sym))
                r0 += n
            biases = [l.bias for l in leaves]
        else:
            w = torch.cat([l.weight.detach() for l in leaves], 0)
            self.base = w
            r0 = 0
            for l in leaves:
                n = l.out_features
                l.weight = nn.Parameter(w[r0:r0 + n], requires_grad=False)
                r0 += n
            biases = [l.bias for l in leaves]
        self.bias = None
        if any(b is not None for b in biases):
            self.bias = torch.cat([b.detach() if b is not None else torch.zeros(n, dtype=self.dtype, device=self.device)
                                   for b, n in zip(biases, self.splits)])

    @property
    def dtype(self):
        return self.base.dtype

    @property
    def device(self):
        return self.base.device

    def branches(self, training: bool) -> list[LoraBranch]:
        out, c0 = [], 0
        for m, n in zip(self.mods, self.splits):
            if isinstance(m, LoraLayer) and not m.merged:
                br = m.branch(c0)
                if not training:
                    br.dropout = 0.0
                out.append(br)
            c0 += n
        return out

    def __call__(self, x, residual=None, training: bool = True):
        if isinstance(self.base, Int4Weight):
            y = int4_linear(x, self.base, self.bias, residual)
            for br in self.branches(False):       # inference-only base: unmerged adapters as plain low-rank adds
                y2 = y.view(-1, y.shape[-1])
                y2[:, br.c0:br.c1] += ((x.reshape(-1, x.shape[-1]) @ br.a.t().to(x.dtype)) @ br.b.t().to(x.dtype)) * br.scaling
            return _apply_multi_lora(self.mods, self.splits, x, y)
        y = fused_linear(x, self.base, self.bias, self.branches(training), residual, training)
        return _apply_multi_lora(self.mods, self.splits, x, y)


def _apply_multi_lora(mods, splits, x, y):
    """Per-request adapters of multi-LoRA serving (``peft/multi_lora.py``): y[:, c0:c1] += the
    row-masked stacked low-rank term of each projection that carries adapters."""
    slots = [getattr(_leaf_linear(m), "_mlora", None) for m in mods]
    if not any(s is not None for s in slots):
        return y
    x2, y2 = x.reshape(-1, x.shape[-1]), y.view(-1, y.shape[-1])
    c0 = 0
    for s, n in zip(slots, splits):
        if s is not None:
            s.apply_(x2, y2, c0)
        c0 += n
    return y


def project(mods: list[nn.Module], x: torch.Tensor, residual: torch.Tensor | None = None,
            training: bool = True, fused: FusedProjection | None = None) -> torch.Tensor:
    """Run projections that share input ``x`` and concatenate their outputs."""
    if fused is not None:
        return fused(x, residual, training)
    if len(mods) == 1:
        m = mods[0]
        if isinstance(m, Int4Linear):            # o_proj / down_proj of a W4A16 model: residual in the epilogue
            y = int4_linear(x.to(torch.bfloat16) if x.is_cuda else x, m.int4, m.bias, residual)
            return _apply_multi_lora(mods, [m.out_features], x, y)
        if _trainable_base(m) or not isinstance(_leaf_linear(m), (nn.Linear, Linear4bit)):
            y = m(x)
            y = _apply_multi_lora(mods, [y.shape[-1]], x, y)
            return y if residual is None else y + residual
        base, bias = base_of(m)
        br = [m.branch()] if isinstance(m, LoraLayer) and not m.merged else []
        if br and not training:
            br[0].dropout = 0.0
        cd = base.dtype if isinstance(base, torch.Tensor) else base.dtype
        y = fused_linear(x.to(cd), base, bias, br, residual, training)
        return _apply_multi_lora(mods, [_out_features(m)], x, y)
    ys = [project([m], x, None, training) for m in mods]
    y = torch.cat(ys, -1)
    return y if residual is None else y + residual


def can_fuse(mods: list[nn.Module]) -> bool:
    leaves = [_leaf_linear(m) for m in mods]
    if any(_trainable_base(m) for m in mods):
        return False
    if all(isinstance(l, Linear4bit) for l in leaves):
        k = leaves[0].in_features
        return all(l.in_features == k and (l.out_features * l.in_features // l.blocksize) % 256 == 0 for l in leaves)
    if all(isinstance(l, Int4Linear) for l in leaves):
        return len({(l.in_features, l.group_size, l.sym) for l in leaves}) == 1
    if all(isinstance(l, nn.Linear) for l in leaves):
        return len({l.in_features for l in leaves}) == 1 and len({l.weight.dtype for l in leaves}) == 1
    return False


class PackedPrefill:
    """Prefill of several prompts packed back to back — ``[1, T]`` tokens, no padding — straight
    into their KV-cache slots (the serving engine's admission path).

    Every token-wise op (projections, norms, SwiGLU: nearly all prefill FLOPs) runs on the
    packed tokens only; attention scatters q/k/v into a right-padded ``[B, S]`` view for the
    flash kernel (causal, per-row ``kv_lens``) and gathers the valid rows back, and each
    layer's K/V rows are written into the cache slots with one indexed copy.  Against padding
    every prompt to the longest one this removes the padded GEMM work (≈ 40 % on chat-length
    prompts) and the scratch-cache → slot copy."""

    def __init__(self, cache: "KVCache", slots: list[int], lens: list[int], device):
        self.cache, self.B, self.S = cache, len(lens), max(lens)
        self.len, self.pos = 0, None              # KVCache duck-typing: a prefill from position 0
        tb = torch.cat([torch.full((n,), b, dtype=torch.long) for b, n in enumerate(lens)])
        tp = torch.cat([torch.arange(n, dtype=torch.long) for n in lens])
        sl = torch.tensor(slots, dtype=torch.long)
        self.positions = tp.to(device)[None]
        self.pad_idx = (tb * self.S + tp).to(device)
        self.cache_idx = (sl[tb] * cache.max_len + tp).to(device)
        self.kv_lens = torch.tensor(lens, dtype=torch.int32, device=device)
        self.last = (torch.cumsum(torch.tensor(lens), 0) - 1).to(device)

    def attend(self, layer: int, q, k, v, hq: int, hkv: int, d: int, attention_fn):
        self.cache.k[layer].view(-1, hkv * d).index_copy_(0, self.cache_idx, k)
        self.cache.v[layer].view(-1, hkv * d).index_copy_(0, self.cache_idx, v)
        if self.B == 1:
            return attention_fn(q, k, v, 1, self.S, hq, hkv, d, causal=True, kv_lens=None)
        n = self.B * self.S

        def pad(t):
            out = t.new_zeros(n, t.shape[1])
            return out.index_copy_(0, self.pad_idx, t)
        o = attention_fn(pad(q), pad(k), pad(v), self.B, self.S, hq, hkv, d, causal=True, kv_lens=self.kv_lens)
        return o.index_select(0, self.pad_idx)


class KVCache:
    """Contiguous pre-allocated KV cache ``[B, Smax, Hkv*D]`` per layer (K17).

    Prefill writes a uniform prefix (``update``; rows may be right-padded, their valid lengths
    live in ``lens``); decode appends one token per row at its own position ``pos[b]``
    (``write_rows``), so a batch of prompts of different lengths decodes without re-padding.
    ``pos`` is a device tensor, so a decode step has no host sync (hipGraph-capturable)."""

    def __init__(self, n_layers: int, batch: int, max_len: int, hkv: int, d: int, dtype, device):
        self.k = [torch.zeros(batch, max_len, hkv * d, dtype=dtype, device=device) for _ in range(n_layers)]
        self.v = [torch.zeros(batch, max_len, hkv * d, dtype=dtype, device=device) for _ in range(n_layers)]
        self.len = 0
        self.max_len = max_len
        self.batch = batch
        self.pos: torch.Tensor | None = None      # [B] int64 next write position (decode mode)
        self._rows = torch.arange(batch, device=device)

    def update(self, layer: int, k: torch.Tensor, v: torch.Tensor, start: int):
        """k/v [B, s, Hkv*D] written at ``start``; returns views up to start+s."""
        s = k.shape[1]
        self.k[layer][:, start:start + s] = k
        self.v[layer][:, start:start + s] = v
        return self.k[layer][:, :start + s], self.v[layer][:, :start + s]

    def write_rows(self, layer: int, k: torch.Tensor, v: torch.Tensor):
        """k/v [B, Hkv*D] written at row-specific positions ``pos``."""
        self.k[layer][self._rows, self.pos] = k
        self.v[layer][self._rows, self.pos] = v

    def head_rows(self, n: int) -> "KVCache":
        """View of the first ``n`` rows sharing storage (and ``pos``) with this cache — the serving
        engine decodes only up to its highest occupied slot."""
        if n == self.batch:
            return self
        v = KVCache.__new__(KVCache)
        v.k = [t[:n] for t in self.k]
        v.v = [t[:n] for t in self.v]
        v.len, v.max_len, v.batch = self.len, self.max_len, n
        v.pos = self.pos[:n] if self.pos is not None else None
        v._rows = self._rows[:n]
        return v

    def packed(self, slots: list[int], lens: list[int], device=None) -> "PackedPrefill":
        """Prompts packed back to back, prefilled straight into ``slots`` (the engine's admission path)."""
        return PackedPrefill(self, slots, lens, device or self.k[0].device)

    def slot_view(self, slot: int, length: int, n: int = 0) -> "KVCache":
        """One slot as a batch-1 cache that already holds ``length`` tokens (chunked / suffix prefill)."""
        view = KVCache.__new__(KVCache)
        view.k = [t[slot:slot + 1] for t in self.k]
        view.v = [t[slot:slot + 1] for t in self.v]
        view.len, view.max_len, view.batch, view.pos = length, self.max_len, 1, None
        view._rows = self._rows[:1]
        return view

    def start_decode(self, lens: torch.Tensor):
        self.pos = lens.to(torch.long).clone()

    def get_seq_length(self) -> int:
        return self.len


class SeqBatch:
    """One engine step over a :class:`SeqStateCache`: the step's tokens packed back to back ``[1, T]`` plus, for each
    sequence in it, its state slot and the position of its first token in this step.

    A fresh prompt starts at 0 (its slot's old state is ignored), a continued prompt or a decode step starts where
    the slot's sequence stands.  Kernels take :attr:`desc` — ``[seq_off (B+1), slots (B), pos0 (B), tok_seq (T),
    tok_pos (T)]`` int32 on the device — and :attr:`live` (``[B]`` int32 or ``None``: rows whose state must not be
    touched carry 0).  ``positions`` / ``last`` mirror :class:`PackedPrefill` for the engine."""

    def __init__(self, cache: "SeqStateCache", desc, host, live=None, max_pos: int | None = None, T: int = 0,
                 tiles=None):
        self.cache, self.desc, self._host, self.live = cache, desc, host, live
        self.tiles = tiles or []          # [tile_seq, tile_t0]: runs of <= 32 tokens of one sequence (attention tiles)
        self.B, self.T = int(desc[1].numel()), T
        self.max_pos = cache.max_len if max_pos is None else max_pos      # bound on any key position this step
        self.decode = host is None
        self.positions = desc[4][None]
        self.len, self.pos = 0, None                                      # KVCache duck-typing (unused)
        self.cache_idx = desc[1].long()[desc[3].long()] * cache.max_len + desc[4].long()
        self.last = (desc[0][1:] - 1).long()

    @classmethod
    def packed(cls, cache: "SeqStateCache", slots: list[int], lens: list[int], starts: list[int] | None = None):
        starts = list(starts) if starts is not None else [0] * len(lens)
        assert len(slots) == len(lens) == len(starts) and all(n > 0 for n in lens)
        if any(s < 0 or s >= cache.batch for s in slots) or len(set(slots)) != len(slots):
            raise ValueError(f"slots {slots}: each must be a distinct row of the cache (0..{cache.batch - 1})")
        if any(p + n > cache.max_len for p, n in zip(starts, lens)):
            raise ValueError(f"a sequence would pass the cache's {cache.max_len} positions")
        off = [0]
        for n in lens:
            off.append(off[-1] + n)
        tok_seq = torch.cat([torch.full((n,), b, dtype=torch.int32) for b, n in enumerate(lens)])
        tok_pos = torch.cat([torch.arange(p, p + n, dtype=torch.int32) for p, n in zip(starts, lens)])
        tile_seq = [b for b, n in enumerate(lens) for _ in range(0, n, 32)]
        tile_t0 = [off[b] + i for b, n in enumerate(lens) for i in range(0, n, 32)]
        flat = torch.cat([torch.tensor(off + list(slots) + starts + tile_seq + tile_t0, dtype=torch.int32), tok_seq, tok_pos])
        flat = flat.to(cache.device)
        B, T, nt = len(lens), off[-1], len(tile_seq)
        parts = list(torch.split(flat, [B + 1, B, B, nt, nt, T, T]))
        desc = parts[:3] + parts[5:]
        return cls(cache, desc, (off, list(slots), starts), None, max(p + n for p, n in zip(starts, lens)), T, parts[3:5])

    @classmethod
    def decoding(cls, cache: "SeqStateCache", n: int):
        """Rows ``[0, n)`` each advance by one token from ``cache.pos`` (a device tensor: no host sync, capturable)."""
        ar = cache._arange[:n + 1]
        pos = cache.pos[:n]
        return cls(cache, [ar, ar[:n], pos, ar[:n], pos], None, cache.live[:n], None, n, [ar[:n], ar[:n]])

    def host(self):
        if self._host is None:      # decode rows on the CPU path: read the positions back
            n = self.B
            return list(range(n + 1)), list(range(n)), [int(p) for p in self.desc[2].tolist()]
        return self._host

    def is_live(self, b: int) -> bool:
        return self.live is None or bool(self.live[b])


class SeqStateCache:
    """Per-slot sequence state for models whose layers are not all plain attention: every layer names the tensors
    it keeps per sequence — K/V rows ``[slots, max_len, C]`` for attention, recurrent matrices and the carried inputs
    of short convolutions ``[slots, ...]`` — and the cache allocates them for ``batch`` slots, like :class:`KVCache`
    does for K/V alone.  ``pos`` (int32, device) is each slot's next position; a slot is recycled by starting its
    next sequence at position 0, which makes every kernel ignore what the slot held.

    ``specs``: per layer a dict ``name -> (shape after the slot axis, "act" | "f32" | "i32" | "kv")``; ``"kv"`` entries
    get the ``max_len`` axis and, like ``"act"`` ones, the activation dtype; ``"i32"`` entries hold integers (a carried
    token).  A model may append dicts of its own after the layers' (state that belongs to no layer)."""

    def __init__(self, specs: list[dict], batch: int, max_len: int, dtype, device):
        self.specs, self.batch, self.max_len, self.dtype, self.device = specs, batch, max_len, dtype, torch.device(device)
        self.layers: list[dict[str, torch.Tensor]] = []
        for spec in specs:
            d = {}
            for name, (shape, kind) in spec.items():
                full = (batch, max_len, *shape) if kind == "kv" else (batch, *shape)
                d[name] = torch.zeros(full, dtype={"f32": torch.float32, "i32": torch.int32}.get(kind, dtype), device=device)
            self.layers.append(d)
        self.pos = torch.zeros(batch, dtype=torch.int32, device=device)
        self.live = torch.ones(batch, dtype=torch.int32, device=device)    # rows whose state a decode step may touch
        self.len = 0
        self.decoding = False             # generate(): set by start_decode, rows then advance one token per call
        self.decode_splits = 1            # key splits of decode attention (fixed per cache: graph-capturable)
        self._arange = torch.arange(batch + 1, dtype=torch.int32, device=device)

    @staticmethod
    def slot_bytes(specs: list[dict], max_len: int, dtype) -> int:
        import math
        el = torch.finfo(dtype).bits // 8
        return sum(math.prod(shape) * (max_len * el if kind == "kv" else el if kind == "act" else 4)   # f32 / i32: 4
                   for spec in specs for shape, kind in spec.values())

    # ---- the views the engine and generate() ask a cache for
    def packed(self, slots: list[int], lens: list[int], device=None) -> SeqBatch:
        return SeqBatch.packed(self, slots, lens)

    def slot_view(self, slot: int, length: int, n: int) -> SeqBatch:
        """``n`` more tokens of the sequence in ``slot`` that already holds ``length``."""
        return SeqBatch.packed(self, [slot], [n], [length])

    def head_rows(self, n: int) -> SeqBatch:
        return SeqBatch.decoding(self, n)

    def set_live(self, rows: list[int], n: int):
        """Decode steps run rows ``[0, n)``; only ``rows`` may change their state (idle rows and rows in the middle
        of a chunked prefill must not)."""
        mask = torch.zeros(self.batch, dtype=torch.int32)
        mask[rows] = 1
        self.live.copy_(mask.to(self.device), non_blocking=True)

    def start_decode(self, lens: torch.Tensor):
        self.pos = lens.to(torch.int32).clone()
        self.decoding = True

    def get_seq_length(self) -> int:
        return self.len


class SeqStateModel(nn.Module):
    """The trunk of a causal LM whose sequences live in a :class:`SeqStateCache`.  A subclass gives
    :meth:`state_specs` and :meth:`run` (packed tokens -> final-normed hidden states); this class turns the calls
    of the serving engine (a :class:`SeqBatch`), of ``generate()`` (right-padded prompts, then one token per row)
    and a plain forward into ``run`` over the right batch view."""

    dtype: torch.dtype
    split_keys = 128          # decode attention: one key split per this many cache positions (at most 32)

    def state_specs(self) -> list[dict]:
        raise NotImplementedError

    def run(self, tokens: torch.Tensor, sb: SeqBatch) -> torch.Tensor:
        raise NotImplementedError

    def state_device(self):
        return next(self.parameters()).device

    def make_cache(self, batch: int, max_len: int, device=None) -> SeqStateCache:
        cache = SeqStateCache(self.state_specs(), batch, max_len, self.dtype, device or self.state_device())
        cache.decode_splits = max(1, min(32, max_len // self.split_keys))     # fixed per cache: graph-capturable
        return cache

    def forward(self, input_ids, position_ids=None, cache=None, kv_lens=None):
        B, S = input_ids.shape
        if isinstance(cache, SeqBatch):                   # the engine's packed prefill / decode rows / chunk
            h = self.run(input_ids.reshape(-1), cache)
            if cache.decode:
                cache.desc[2].add_(1)                     # cache.pos[:n], in place (graph-capturable)
            return h
        if cache is None:
            cache = self.make_cache(B, S, input_ids.device)
        if getattr(cache, "decoding", False) and S == 1:  # generate(): every row one token further
            sb = cache.head_rows(B)
            h = self.run(input_ids.reshape(-1), sb)
            sb.desc[2].add_(1)
            return h
        # generate() / plain forward: right-padded prompts, all from the cache's common length
        lens = [S] * B if kv_lens is None else [int(n) for n in kv_lens.tolist()]
        start = cache.len
        sb = SeqBatch.packed(cache, list(range(B)), lens, [start] * B)
        keep = (torch.arange(S, device=input_ids.device)[None] <
                torch.tensor(lens, device=input_ids.device)[:, None]).reshape(-1)
        hp = self.run(input_ids.reshape(-1)[keep], sb)
        cache.len = start + S
        if all(n == S for n in lens):
            return hp
        h = hp.new_zeros(B * S, hp.shape[1])
        h[keep] = hp
        return h


class _HeadWeight(nn.Module):
    def __init__(self, w):
        super().__init__()
        self.weight = nn.Parameter(w, requires_grad=False)


class SeqStateCausalLM(nn.Module):
    """``.model`` (a :class:`SeqStateModel`) + ``.lm_head`` like the other causal LMs, so ``infer.generate`` and the
    serving engine drive it; the engine asks :meth:`make_cache` for its slot pool and :meth:`compute_logits` for
    logits.  A subclass sets ``config_class`` (``from_pretrained(path)`` / ``from_dict``) and builds ``self.model`` and
    ``self.lm_head`` from ``(config, weights by checkpoint name, dtype, device)``."""

    config_class = None
    logit_scale = 1.0

    @classmethod
    def from_pretrained(cls, path: str, dtype=torch.bfloat16, device=None, **_):
        import os
        from safetensors import safe_open
        cfg = cls.config_class.from_pretrained(path)
        W = {}
        for f in sorted(f for f in os.listdir(path) if f.endswith(".safetensors")):
            with safe_open(os.path.join(path, f), framework="pt", device="cpu") as fh:
                for k in fh.keys():
                    W[k] = fh.get_tensor(k)
        return cls(cfg, W, dtype, device)

    def make_cache(self, batch: int, max_len: int, device=None) -> SeqStateCache:
        return self.model.make_cache(batch, max_len, device)

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        """Float logits ``head h * logit_scale`` (bf16 products accumulate in float and are not rounded back)."""
        w = self.lm_head.weight
        h2 = h.reshape(-1, h.shape[-1])
        if w.dtype == torch.float32 or not h2.is_cuda:
            y = h2.float() @ w.float().t()
        else:
            y = torch.mm(h2, w.t(), out_dtype=torch.float32)
        if self.logit_scale != 1.0:
            y = y * self.logit_scale
        return y.view(*h.shape[:-1], w.shape[0])

    def forward(self, input_ids, attention_mask=None, labels=None, past_key_values=None, **_) -> CausalLMOutput:
        B, S = input_ids.shape
        kv_lens = attention_mask.sum(1) if attention_mask is not None else None
        with torch.no_grad():
            h = self.model(input_ids, None, past_key_values, kv_lens)
            logits = self.compute_logits(h).view(B, S, -1)
        loss = None
        if labels is not None:
            loss = torch.nn.functional.cross_entropy(logits[:, :-1].reshape(-1, logits.shape[-1]).float(),
                                                     labels[:, 1:].reshape(-1), ignore_index=-100)
        return CausalLMOutput(loss=loss, logits=logits, past_key_values=past_key_values)

    @torch.no_grad()
    def generate(self, input_ids=None, attention_mask=None, generation_config=None, streamer=None, **kw):
        from ..infer.generate import generate
        return generate(self, input_ids, attention_mask, generation_config, streamer=streamer, **kw)
