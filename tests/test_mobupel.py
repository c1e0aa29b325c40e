"""Mobupel on the framework (packed batches, slot state, engine step functions, HIP kernels on a GPU) against the
plain float64 implementation of tests/mobupel_oracle.py.  Every test makes its own small configuration and weights;
each runs on the CPU path and, marked ``gpu``, on the HIP kernels."""
import copy
import queue

import pytest
import torch

import mobupel_oracle as O
from llm_in_practise_amd.infer.engine import SamplingParams, ServingEngine
from llm_in_practise_amd.infer.trace import TraceRunner
from llm_in_practise_amd.models.common import SeqBatch
from llm_in_practise_amd.models.mobupel import MobupelConfig, MobupelForCausalLM

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def mlstm(heads=3, dim=8, vdim=20, cap=10.0, mlp=None):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap},
            "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def parallel(lh=6, lg=3, ldim=16, lvdim=8, lconv=3, scale=0.3, rh=4, rg=2, rdim=8, rvdim=12, rconv=2, mlp=40):
    left = {"heads": lh, "kv_heads": lg, "dim": ldim, "vdim": lvdim, "scale": scale}
    if lconv:
        left["conv"] = lconv
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rh, "kv_heads": rg, "dim": rdim, "vdim": rvdim,
                                                                  "conv": rconv}},
            "mlp": None if mlp is None else {"kind": "dense", "ff": mlp}}


def config(layers, width=48, vocab=61, eps=1e-5, escale=3.0, lscale=0.7, **extra):
    return {"architecture": "Mobupel", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "embedding": {"scale": escale}, "logit_scale": lscale, **extra}


BASE = config([parallel(), mlstm(), mlstm(heads=2, dim=24, vdim=6, cap=4.0, mlp=24), parallel(mlp=None, lconv=5, rconv=4)])


def build(cfg, device, seed=0, dtype=torch.float32, tweak=None):
    W = O.random_weights(cfg, seed)
    if tweak:
        tweak(W)
    if dtype == torch.bfloat16:
        W = {k: v.to(torch.bfloat16).float() for k, v in W.items()}
    lm = MobupelForCausalLM(MobupelConfig.from_dict(cfg), W, dtype, device)
    return lm, W


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def close(got, want, tol=2e-4):
    got, want = got.double().cpu(), want.double()
    err = (got - want).abs().max().item() / max(want.abs().max().item(), 1e-9)
    assert err < tol, f"relative error {err:.3g}"


def replay(lm, max_tokens, steps):
    """steps: list of (entries, end); every entry asks for all its tokens.  Returns {id: logits [n, vocab]}."""
    r, out = TraceRunner(lm, max_tokens), {}
    for entries, end in steps:
        es = [{"id": i, "tokens": t, "want": list(range(len(t)))} for i, t in entries]
        got = r.step(es, end)
        o = 0
        for i, t in entries:
            out[i] = torch.cat([out[i], got[o:o + len(t)]]) if i in out else got[o:o + len(t)]
            o += len(t)
    return out


# --------------------------------------------------------------------------------------- each mechanism alone
def _one_layer(device, layer, T=19, tweak=None, seed=1, **kw):
    cfg = config([layer], **kw)
    lm, W = build(cfg, device, seed, tweak=tweak)
    toks = tokens(T, cfg["vocab"], seed)
    got = replay(lm, T, [([("a", toks)], ["a"])])["a"]
    close(got, O.forward(cfg, W, toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("heads,dim,vdim,cap", [(3, 8, 20, 10.0), (1, 40, 72, 2.0), (2, 16, 16, 30.0)])
def test_mlstm_alone(device, heads, dim, vdim, cap):
    _one_layer(device, mlstm(heads, dim, vdim, cap), T=40)


def _silence(side):
    def tweak(W):
        W[f"l0.mix.{side}.o"].zero_()
    return tweak


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(lh=4, lg=1, ldim=12, lvdim=80, lconv=1), dict(lh=2, lg=2, lconv=0, scale=2.5),
                                dict(lh=8, lg=2, ldim=8, lvdim=8, lconv=7)])
def test_talking_heads_attention_alone(device, kw):
    _one_layer(device, parallel(**kw), T=33, tweak=_silence("right"))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(rh=6, rg=1, rdim=20, rvdim=5, rconv=3), dict(rh=2, rg=2, rdim=48, rvdim=70, rconv=1)])
def test_gated_delta_rule_alone(device, kw):
    _one_layer(device, parallel(**kw), T=33, tweak=_silence("left"))


@pytest.mark.parametrize("device", DEVICES)
def test_feed_forward_and_gated_residual(device):
    _one_layer(device, mlstm(mlp=56), T=9, width=40, eps=1e-3)


@pytest.mark.parametrize("device", DEVICES)
def test_short_conv_carries_inputs(device):
    """Convolution over a sequence cut into pieces of 1..5 tokens equals the whole, for every tail mode."""
    from llm_in_practise_amd.models.common import SeqStateCache
    from llm_in_practise_amd.ops import conv as C
    g = torch.Generator().manual_seed(3)
    T, taps, heads, hw = 23, 4, 3, 10
    Cn = 3 * heads * hw
    u, w, nw = torch.randn(T, Cn, generator=g), torch.randn(Cn, taps, generator=g), torch.rand(hw, generator=g) + 0.5
    want = O.short_conv(u.double(), w.double()).view(T, 3, heads, hw)
    want[:, 0] = O.rms_norm(want[:, 0], nw.double(), 1e-5)
    sl = torch.nn.functional.silu(want[:, 2])
    want[:, 2] = sl / torch.sqrt((sl * sl).sum(-1, keepdim=True) + 1e-6) * 0.5
    segs = [(0, heads, hw, C.RMS, nw.to(device), 1.0), (heads * hw, heads, hw, C.PLAIN, None, 1.0),
            (2 * heads * hw, heads, hw, C.SILU_UNIT, None, 0.5)]
    cache = SeqStateCache([{"c": ((taps - 1, Cn), "act")}], 3, 64, torch.float32, device)
    cache.layers[0]["c"].fill_(7.0)                     # a used slot: must not leak into a fresh sequence
    got, p = [], 0
    for n in (1, 1, 2, 5, 3, 1, 4, 6):
        sb = SeqBatch.packed(cache, [1], [n], [p])
        got.append(C.short_conv(u[p:p + n].to(device), w.to(device), cache.layers[0]["c"], segs, sb, 1e-5, out_f32=True))
        p += n
    close(torch.cat(got), want.reshape(T, Cn), 1e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_embedding_positions(device):
    from llm_in_practise_amd.ops.embedding import embed_sincos, sinusoid_inv_freq
    g = torch.Generator().manual_seed(5)
    table = torch.randn(17, 30, generator=g)
    tok = torch.tensor([3, 16, 0, 5])
    want = O.embed(tok, table.double(), 2.5, 30, start=700)
    got = embed_sincos(tok.to(device), torch.arange(700, 704, dtype=torch.int32, device=device), table.to(device),
                       sinusoid_inv_freq(30).to(device), 2.5)
    close(got, want, 2e-5)


# --------------------------------------------------------------- whole prompts, decoding, portions, batches, slots
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(device):
    lm, W = build(BASE, device)
    toks = tokens(26, BASE["vocab"], 2)
    want = O.forward(BASE, W, toks)
    close(replay(lm, 40, [([("a", toks)], ["a"])])["a"], want)
    steps = [([("a", toks[:1])], [])] + [([("a", [t])], []) for t in toks[1:]]
    close(replay(lm, 40, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [(2, 2, 2, 20), (7, 3, 2, 14), (1, 24, 1), (13, 13)])
def test_portions(device, cuts):
    lm, W = build(BASE, device)
    toks = tokens(sum(cuts), BASE["vocab"], 3)
    steps, p = [], 0
    for n in cuts:
        steps.append(([("a", toks[p:p + n])], []))
        p += n
    close(replay(lm, 40, steps)["a"], O.forward(BASE, W, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(device):
    lm, W = build(BASE, device)
    V = BASE["vocab"]
    seqs = {"a": tokens(31, V, 4), "b": tokens(5, V, 5), "c": tokens(1, V, 6), "d": tokens(17, V, 7)}
    tail = {k: tokens(9, V, 10 + i) for i, k in enumerate(seqs)}
    tail["b"] = tail["b"][:3]                        # ends early, the batch goes on without it
    steps = [([(k, v) for k, v in seqs.items()], [])]
    for j in range(9):
        live = [k for k in seqs if j < len(tail[k])]
        steps.append(([(k, [tail[k][j]]) for k in live], [k for k in live if j == len(tail[k]) - 1]))
    got = replay(lm, 200, steps)
    for k in seqs:
        close(got[k], O.forward(BASE, W, seqs[k] + tail[k]))


@pytest.mark.parametrize("device", DEVICES)
def test_slots_freed_and_reused(device):
    lm, W = build(BASE, device)
    V = BASE["vocab"]
    a, b, c, d = tokens(30, V, 8), tokens(11, V, 9), tokens(4, V, 10), tokens(21, V, 11)
    steps = [([("a", a), ("b", b)], ["a"]),          # a's slot (0) is free again, b lives on in slot 1
             ([("c", c[:3])], []),                   # c takes slot 0 over a's longer state
             ([("c", [c[3]]), ("b", [b[0]])], ["c", "b"]),
             ([("d", d)], ["d"])]
    got = replay(lm, 80, steps)
    close(got["a"], O.forward(BASE, W, a))
    close(got["c"], O.forward(BASE, W, c))
    close(got["d"], O.forward(BASE, W, d))
    close(got["b"], O.forward(BASE, W, b + [b[0]]))


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    cfg = config([mlstm(cap=3.0), parallel(mlp=16, lconv=6, rconv=5)], width=32)
    lm, W = build(cfg, device, seed=4)
    toks = tokens(150, cfg["vocab"], 12)
    steps = [([("a", toks[:2])], [])] + [([("a", [t])], []) for t in toks[2:]]
    got = replay(lm, 160, steps)["a"]
    want = O.forward(cfg, W, toks)
    close(got[:8], want[:8])
    close(got, want, 5e-4)


# ------------------------------------------------------------------------- keys far away, made to stand out
def _needle_weights(W, cfg, width):
    """Left attention reads (almost) only the token's embedding direction: q = k = a scaled copy of the input, no
    convolution mixing (taps weight on the current token), so a query finds the earlier position with its own token."""
    p = "l0.mix.left."
    m = cfg["layers"][0]["mixer"]["left"]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    eye = torch.eye(dk, width)
    W[p + "q"] = eye.repeat(H, 1) * 6.0
    W[p + "k"] = eye.repeat(G, 1) * 6.0
    for n in "qkv":
        W[p + n + ".conv"].zero_()
        W[p + n + ".conv"][:, -1] = 1.0
    W["l0.mix.right.o"].zero_()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T", [130, 700])
def test_far_key_stands_out(device, T):
    """Early tokens recur at the end: their keys far back take a large share of the softmax, in a prompt and in
    decoding, across the 64-key sweeps and — for the long case — the key splits of decode attention."""
    width = 32
    cfg = config([parallel(lh=4, lg=2, ldim=16, lvdim=8, lconv=2, scale=1.0, mlp=None)], width=width, vocab=97,
                 escale=30.0)                          # embeddings outweigh the position vector: same token, same key
    lm, W = build(cfg, device, seed=6, tweak=lambda W: _needle_weights(W, cfg, width))
    toks = [t % 90 for t in tokens(T, 90, 13)]
    for far in (0, 1, 63, 64, 65, T - 70):
        toks[far] = 90 + (far % 7)                    # rare tokens planted far back ...
    probe = [90, 91, 90 + 63 % 7, 90 + 64 % 7, 90 + 65 % 7, 90 + (T - 70) % 7]
    full = toks + probe                               # ... and asked for again at the end
    want = O.forward(cfg, W, full)
    close(replay(lm, 1100, [([("a", full)], ["a"])])["a"], want)
    steps = [([("a", toks)], [])] + [([("a", [t])], []) for t in probe]
    close(replay(lm, 1100, steps)["a"], want)
    # the planted key matters: without it the answer differs by far more than the tolerance
    other = list(full)
    other[64] = 5
    assert (O.forward(cfg, W, other)[-3] - want[-3]).abs().max() > 1e-2 * want[-3].abs().max()


@pytest.mark.parametrize("device", DEVICES)
def test_recurrent_memory_of_far_token(device):
    """A slowly forgetting delta-rule head keeps a token written hundreds of steps back."""
    cfg = config([parallel(rh=2, rg=1, rdim=16, rvdim=16, rconv=2, mlp=None)], width=32)

    def tweak(W):
        W["l0.mix.left.o"].zero_()
        W["l0.mix.right.A_log"].fill_(-9.0)           # decay ~ exp(-1e-4 * softplus): almost none
    lm, W = build(cfg, device, seed=7, tweak=tweak)
    toks = tokens(400, cfg["vocab"], 14)
    want = O.forward(cfg, W, toks)
    steps = [([("a", toks[:380])], [])] + [([("a", [t])], []) for t in toks[380:]]
    close(replay(lm, 410, steps)["a"], want, 5e-4)
    other = list(toks)
    other[3] = (other[3] + 1) % cfg["vocab"]
    assert (O.forward(cfg, W, other)[-1] - want[-1]).abs().max() > 1e-3 * want[-1].abs().max()


# ------------------------------------------------------------------------------ other sizes, degenerate values
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [
    config([mlstm(heads=1, dim=8, vdim=8, mlp=8)], width=16, vocab=11, escale=1.0, lscale=1.0),
    config([parallel(lh=1, lg=1, ldim=8, lvdim=8, lconv=1, scale=1.0, rh=1, rg=1, rdim=8, rvdim=8, rconv=1, mlp=None)],
           width=8, vocab=9),
    config([parallel(lh=4, lg=4, ldim=24, lvdim=40, lconv=8, rh=3, rg=3, rdim=40, rvdim=24, rconv=8)] * 2
           + [mlstm(heads=5, dim=12, vdim=12)], width=72, vocab=130, _rank_a=3, _rank_g=11),
])
def test_other_sizes(device, cfg):
    lm, W = build(cfg, device, seed=8)
    a, b = tokens(14, cfg["vocab"], 15), tokens(6, cfg["vocab"], 16)
    got = replay(lm, 40, [([("a", a[:9]), ("b", b[:4])], []), ([("a", [a[9]]), ("b", [b[4]])], []),
                          ([("a", [a[10]]), ("b", [b[5]])], ["b"]), ([("a", a[11:])], ["a"])])
    close(got["a"], O.forward(cfg, W, a))
    close(got["b"], O.forward(cfg, W, b))


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_weights_and_activations(device):
    lm, W = build(BASE, device, dtype=torch.bfloat16)
    toks = tokens(40, BASE["vocab"], 17)
    got = replay(lm, 60, [([("a", toks[:30])], [])] + [([("a", [t])], []) for t in toks[30:]])["a"]
    close(got, O.forward(BASE, W, toks), 0.06)


def test_checkpoint_roundtrip_and_registry(tmp_path):
    import json
    from safetensors.torch import save_file
    from llm_in_practise_amd.models.registry import load_causal_lm
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in O.random_weights(BASE, 9).items()}
    save_file(W, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps({k: v for k, v in BASE.items() if not k.startswith("_")}))
    lm = load_causal_lm(str(tmp_path), dtype=torch.float32, device="cpu")
    assert type(lm).__name__ == "MobupelForCausalLM"
    toks = tokens(12, BASE["vocab"], 18)
    close(lm(torch.tensor([toks])).logits[0], O.forward(BASE, W, toks))
    bad = copy.deepcopy(BASE)
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        MobupelConfig.from_dict(bad)


# ------------------------------------------------- greedy generation through the entry points and the scheduler
def _greedy(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(cfg, W, seq)[-1].argmax()))
    return seq[len(prompt):]


class _Tok:
    """Token i <-> chr(0x100 + i): text in, text out, no special tokens."""
    eos_token_id = None
    pad_token_id = 0

    def encode(self, s, add_special_tokens=False):
        return [ord(c) - 0x100 for c in s]

    def decode(self, ids, skip_special_tokens=True):
        return "".join(chr(0x100 + int(i)) for i in ids)


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_engine_and_generate(device):
    cfg = config([mlstm(), parallel(), mlstm(mlp=32)], width=40, vocab=53)
    lm, W = build(cfg, device, seed=10)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (9, 3, 14, 1, 6)]
    want = [_greedy(cfg, W, p, 7) for p in prompts]
    # generate(): right-padded batch of unequal prompts
    S = max(map(len, prompts))
    ids = torch.tensor([p + [0] * (S - len(p)) for p in prompts], device=device)
    mask = torch.tensor([[1] * len(p) + [0] * (S - len(p)) for p in prompts], device=device)
    out = lm.generate(ids, attention_mask=mask, max_new_tokens=7, do_sample=False)
    for b, p in enumerate(prompts):
        assert out[b, len(p):len(p) + 7].tolist() == want[b]
    # the serving engine: a queue, 3 slots for 5 requests (slots are reused), continuous batching
    tok = _Tok()
    eng = ServingEngine(lm, tok, max_batch=3, max_model_len=64, use_graphs=False)
    try:
        reqs = [eng.submit(tok.decode(p), SamplingParams(max_tokens=7, temperature=0.0)) for p in prompts]
        for r, w in zip(reqs, want):
            while True:
                kind, val = r.out.get(timeout=120)
                if kind == "error":
                    raise RuntimeError(val)
                if kind == "final":
                    break
            assert tok.encode(val["text"]) == w
    finally:
        eng.shutdown()
    # chunked prefill through the scheduler: long prompts enter 4 tokens per iteration between decode steps
    eng = ServingEngine(lm, tok, max_batch=2, max_model_len=64, use_graphs=False, chunked_prefill=4)
    try:
        reqs = [eng.submit(tok.decode(p), SamplingParams(max_tokens=7, temperature=0.0)) for p in prompts]
        for r, w in zip(reqs, want):
            kind, val = r.out.get(timeout=120)
            assert kind == "final", val
            assert tok.encode(val["text"]) == w
    finally:
        eng.shutdown()


@pytest.mark.gpu
def test_decode_graphs_replay_equals_eager():
    """Captured decode steps, replayed many times with eager prefills between them, give the eager logits."""
    cfg = config([mlstm(), parallel(), mlstm(mlp=32)], width=40, vocab=53)
    lm, W = build(cfg, "cuda", seed=11)
    V = cfg["vocab"]
    a, b, c = tokens(30, V, 30), tokens(12, V, 31), tokens(20, V, 32)

    def run(graphs):
        r, out = TraceRunner(lm, 200, use_graphs=graphs), {}
        steps = [([("a", a[:10]), ("b", b[:5])], [])] + [([("a", [a[10 + j]]), ("b", [b[5 + j]])], []) for j in range(7)]
        steps[-1] = (steps[-1][0], ["b"])
        steps += [([("c", c[:8])], [])] + [([("a", [a[17 + j]]), ("c", [c[8 + j]])], []) for j in range(12)]
        for entries, end in steps:
            got = r.step([{"id": i, "tokens": t, "want": list(range(len(t)))} for i, t in entries], end)
            o = 0
            for i, t in entries:
                out[i] = torch.cat([out[i], got[o:o + len(t)]]) if i in out else got[o:o + len(t)]
                o += len(t)
        return out
    eager, graph = run(False), run(True)
    for k in eager:
        close(graph[k], eager[k].double(), 1e-5)
    close(eager["a"], O.forward(cfg, W, a[:29]))
    close(eager["c"], O.forward(cfg, W, c))


@pytest.mark.gpu
@pytest.mark.parametrize("dk,dv,H,G", [(32, 32, 4, 2), (64, 128, 6, 3), (144, 160, 2, 1), (128, 64, 8, 8), (64, 64, 8, 2),
                                       (160, 192, 4, 1), (16, 32, 16, 2)])
@pytest.mark.parametrize("scale", [0.2, 4.0])
def test_matrix_core_attention_sweep(dk, dv, H, G, scale):
    """bf16 head-mixing attention on the matrix-core kernel (ragged batch, continued sequences, tiles that end inside
    a sequence, key splits) against per-query float64 sums over the same bf16 inputs; a sharp scale makes single keys
    carry the result."""
    from llm_in_practise_amd.models.common import SeqStateCache
    from llm_in_practise_amd.ops.attention import talking_heads_attention
    g = torch.Generator().manual_seed(dk + dv)
    lens, starts, slots, max_len = [70, 1, 33, 32, 5], [0, 130, 31, 64, 0], [4, 0, 2, 5, 1], 256
    cache = SeqStateCache([{"k": ((G * dk,), "kv"), "v": ((G * dv,), "kv")}], 6, max_len, torch.bfloat16, "cuda")
    kc = torch.randn(6, max_len, G * dk, generator=g).to(torch.bfloat16)
    vc = torch.randn(6, max_len, G * dv, generator=g).to(torch.bfloat16)
    cache.layers[0]["k"].copy_(kc)
    cache.layers[0]["v"].copy_(vc)
    T = sum(lens)
    q = torch.randn(T, H * dk, generator=g).to(torch.bfloat16)
    gate = torch.randn(T, H * dv, generator=g).to(torch.bfloat16)
    talk = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).float()
    sb = SeqBatch.packed(cache, slots, lens, starts)
    for nsplit in (1, 3):
        got = talking_heads_attention(q.cuda(), cache.layers[0]["k"], cache.layers[0]["v"], talk.cuda(), gate.cuda(), H, G,
                                      scale, sb, nsplit).float().cpu()
        t = 0
        for b, n in enumerate(lens):
            for i in range(n):
                L = starts[b] + i + 1
                kk = kc[slots[b], :L].double().view(L, G, dk)
                vv = vc[slots[b], :L].double().view(L, G, dv)
                w = torch.stack([torch.softmax(kk[:, h // (H // G)] @ q[t].double().view(H, dk)[h] * scale, 0) for h in range(H)])
                w = talk.double() @ w
                o = torch.stack([w[h] @ vv[:, h // (H // G)] for h in range(H)]).reshape(-1) * torch.sigmoid(gate[t].double())
                err = (got[t].double() - o).abs().max() / o.abs().max()
                assert err < 2e-2, (b, i, nsplit, float(err))
                t += 1


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_matrix_core_sizes_long_context(device):
    """bf16 model whose attention sizes take the matrix-core path; 600 tokens, then decoding across key splits."""
    cfg = config([parallel(lh=8, lg=2, ldim=32, lvdim=32, lconv=3, scale=0.25, mlp=None),
                  parallel(lh=4, lg=2, ldim=64, lvdim=32, lconv=2, scale=0.125, mlp=32)], width=64)
    lm, W = build(cfg, device, seed=12, dtype=torch.bfloat16)
    toks = tokens(620, cfg["vocab"], 19)
    got = replay(lm, 1100, [([("a", toks[:600])], [])] + [([("a", [t])], []) for t in toks[600:]])["a"]
    close(got, O.forward(cfg, W, toks), 0.06)
