"""Dogudra on the framework (packed batches, slot state, engine step functions, HIP kernels on a GPU) against the
plain float64 implementation of tests/dogudra_oracle.py.  Every test makes its own small configuration and weights;
each runs on the CPU path and, marked ``gpu``, on the HIP kernels."""
import copy
import json

import pytest
import torch

import dogudra_oracle as O
from llm_in_practise_amd.infer.engine import SamplingParams, ServingEngine
from llm_in_practise_amd.infer.trace import TraceRunner
from llm_in_practise_amd.models.common import SeqBatch, SeqStateCache
from llm_in_practise_amd.models.dogudra import DogudraConfig, DogudraForCausalLM

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, identity=1, top=2, count=1, keep=1, scale=1.7, ff=24, limit=1.5, shared=20, shared_limit=2.5):
    r = {"experts": experts, "identity": identity, "top": top, "scale": scale}
    if count > 1:
        r["groups"] = {"count": count, "keep": keep}
    out = {"kind": "moe", "router": r, "expert": {"ff": ff, "limit": limit}}
    if shared:
        out["shared"] = {"ff": shared, "limit": shared_limit}
    return out


def attn(heads=3, dim=8, rot=4, vdim=12, kv_rank=20, q_rank=14, scale=0.3, base=100.0, kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
         "rot": {"base": base, "dims": rot}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def ssm(heads=4, vdim=6, state=10, groups=2, conv=3, norm_groups=2, mlp=None):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}, "mlp": mlp}


def config(layers, width=48, vocab=61, eps=1e-5, escale=2.0, alpha=2.5, bigram=(37, 11, 5)):
    e = {"scale": escale}
    if bigram:
        e["bigram"] = {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}
    return {"architecture": "Dogudra", "width": width, "vocab": vocab, "layers": layers, "norm": {"eps": eps},
            "postln_alpha": alpha, "embedding": e}


BASE = config([attn(mlp=dense()), ssm(mlp=moe(count=1)), attn(kv_from=0, mlp=moe(experts=6, identity=2, top=3, count=4, keep=2)),
               attn(heads=2, dim=16, rot=8, vdim=8, kv_rank=24, q_rank=10, scale=0.2), ssm(heads=2, vdim=16, state=18, groups=1,
                                                                                          conv=4, norm_groups=1, mlp=dense(24)),
               attn(heads=2, dim=16, rot=8, vdim=8, kv_rank=24, q_rank=10, scale=0.2, kv_from=3, mlp=moe(identity=0, shared=0))])


def build(cfg, device, seed=0, dtype=torch.float32, tweak=None):
    W = O.random_weights(cfg, seed)
    if tweak:
        tweak(W)
    if dtype == torch.bfloat16:
        W = {k: v.to(torch.bfloat16).double() for k, v in W.items()}
    lm = DogudraForCausalLM(DogudraConfig.from_dict(cfg), W, dtype, device)
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
def _check(device, layers, T=23, tweak=None, seed=1, decode_from=None, **kw):
    cfg = config(layers, **kw)
    lm, W = build(cfg, device, seed, tweak=tweak)
    toks = tokens(T, cfg["vocab"], seed)
    want = O.forward(toks, W, cfg)
    close(replay(lm, T, [([("a", toks)], ["a"])])["a"], want)
    if decode_from is not None:
        steps = [([("a", toks[:decode_from])], [])] + [([("a", [t])], []) for t in toks[decode_from:]]
        close(replay(lm, T, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=4, rot=2, vdim=40, kv_rank=8, q_rank=3, scale=1.5),
                                dict(heads=5, dim=12, rot=6, vdim=4, kv_rank=16, q_rank=48, base=7.0),
                                dict(heads=2, dim=16, rot=16, vdim=16, kv_rank=32, q_rank=16)])
def test_latent_attention_alone(device, kw):
    _check(device, [attn(**kw)], decode_from=9)


@pytest.mark.parametrize("device", DEVICES)
def test_latent_attention_borrows_cache_of_earlier_layer(device):
    """Two borrowers of layer 0 (one not adjacent), each with its own up-projections; a borrowed cache that was
    rotated once must not be rotated again."""
    _check(device, [attn(), ssm(), attn(kv_from=0), attn(kv_from=0, heads=2, vdim=6, q_rank=9)], decode_from=5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=6, vdim=4, state=5, groups=3, conv=1, norm_groups=3),
                                dict(heads=2, vdim=24, state=40, groups=2, conv=5, norm_groups=1),
                                dict(heads=1, vdim=8, state=16, groups=1, conv=2, norm_groups=4)])
def test_state_space_mixer_alone(device, kw):
    _check(device, [ssm(**kw)], decode_from=4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kw", [dict(), dict(experts=8, identity=0, top=1, count=2, keep=1, shared=0),
                                dict(experts=5, identity=3, top=4, count=4, keep=3, scale=0.6, limit=0.4),
                                dict(experts=2, identity=2, top=4, count=1), dict(experts=9, identity=1, top=2, count=5, keep=1)])
def test_routed_feed_forward(device, kw):
    """Long enough that the prompt takes the sorted path and the decode steps the pair-streaming path."""
    _check(device, [attn(mlp=moe(**kw))], T=45, decode_from=40)


@pytest.mark.parametrize("device", DEVICES)
def test_routed_feed_forward_long_prompt(device):
    """300 tokens in one step (the router kernel's form for many tokens, experts with long runs of rows)."""
    _check(device, [ssm(mlp=moe(experts=4, identity=2, top=3, count=3, keep=2))], T=300)


@pytest.mark.parametrize("device", DEVICES)
def test_dense_feed_forward_and_layer_without_one(device):
    _check(device, [ssm(mlp=dense(56)), attn()], alpha=0.7)


@pytest.mark.parametrize("device", DEVICES)
def test_router_choices(device):
    """Made-up scores: the correction decides the choice but not the weight; a group outside the kept ones loses even
    with the second-best output; negative choice values still beat masked ones."""
    from llm_in_practise_amd.ops.moe import route_grouped
    z = torch.log(torch.tensor([[0.30, 0.05, 0.04, 0.28, 0.20, 0.13],
                                [0.02, 0.03, 0.45, 0.30, 0.12, 0.08]], device=device))
    s = torch.softmax(z, -1).cpu()
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, -0.5, 0.3], device=device)
    # runs {0,1} {2,3} {4,5}, one kept.  Row 0: the largest choice is output 5 (0.13 + 0.3), so output 0 (the best
    # plain score) loses with its run, and output 4 is taken although its choice value is negative (0.2 - 0.5).
    idx, w = route_grouped(z, corr, 2, 3, 1, 2.0)
    assert idx.tolist() == [[5, 4], [2, 3]]
    close(w, 2.0 * s.gather(1, idx.cpu().long()))         # weights: plain scores, scaled, not renormalised
    idx, w = route_grouped(z, None, 3, 3, 2, 1.0)
    assert idx.tolist() == [[0, 3, 1], [2, 3, 4]]
    close(w, s.gather(1, idx.cpu().long()))


@pytest.mark.parametrize("device", DEVICES)
def test_router_ids_stay_in_range_for_any_input(device):
    """Rows nobody reads (idle decode rows) may hold anything; their expert ids must still be usable as addresses."""
    from llm_in_practise_amd.ops.moe import route_grouped, route_tokens
    g = torch.Generator().manual_seed(1)
    h = torch.randn(6, 32, generator=g)
    h[1, 3], h[2, :], h[4, 7] = float("nan"), float("inf"), float("-inf")
    router, corr = torch.randn(10, 32, generator=g).to(device), (0.1 * torch.randn(10, generator=g)).to(device)
    for idx, _ in (route_tokens(h.to(device), router, corr, 3, 2, 1, 1.5), route_grouped(h.to(device)[:, :10].contiguous(), corr, 3)):
        assert int(idx.min()) >= 0 and int(idx.max()) < 10


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("bigram", [(37, 11, 5), (2, 1, 1), (1009, 131, 7), None])
def test_pair_embedding_carries_last_token(device, bigram):
    cfg = config([ssm(conv=1)], bigram=bigram, escale=0.5)
    lm, W = build(cfg, device, seed=3)
    toks = tokens(12, cfg["vocab"], 3)
    want = O.forward(toks, W, cfg)
    for cut in (1, 2, 11):
        close(replay(lm, 20, [([("a", toks[:cut])], []), ([("a", toks[cut:])], ["a"])])["a"], want)
    taps = []
    O.forward(toks, W, cfg, taps)
    lm.model.residual_tap = got = []
    replay(lm, 20, [([("a", toks)], ["a"])])
    close(got[0], taps[0])


@pytest.mark.parametrize("device", DEVICES)
def test_conv_inputs_carried_over_dirty_slot(device):
    from llm_in_practise_amd.ops import conv as C
    from llm_in_practise_amd.ops.conv import short_conv
    g = torch.Generator().manual_seed(5)
    Cn, taps = 24, 4
    u, w, b = torch.randn(11, Cn, generator=g), torch.randn(Cn, taps, generator=g), torch.randn(Cn, generator=g)
    want = torch.nn.functional.silu(O.causal_conv(u.double(), w.double(), b.double()))
    cache = SeqStateCache([{}], 3, 32, torch.float32, device)
    state = torch.full((3, taps - 1, Cn), 7.0, device=device)          # what an earlier sequence left behind
    outs, p = [], 0
    for n in (1, 2, 3, 5):
        sb = SeqBatch.packed(cache, [2], [n], [p])
        outs.append(short_conv(u[p:p + n].to(device), w.to(device), state, [(0, 3, 8, C.SILU, None, 1.0)], sb, 1e-6,
                               bias=b.to(device)))
        p += n
    close(torch.cat(outs), want, 1e-5)


# --------------------------------------------------------------- whole prompts, decoding, portions, batches, slots
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_equals_token_by_token(device):
    lm, W = build(BASE, device)
    toks = tokens(26, BASE["vocab"], 2)
    want = O.forward(toks, W, BASE)
    close(replay(lm, 40, [([("a", toks)], ["a"])])["a"], want)
    steps = [([("a", toks[:1])], [])] + [([("a", [t])], []) for t in toks[1:]]
    close(replay(lm, 40, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_stream_after_every_layer(device):
    lm, W = build(BASE, device)
    toks = tokens(9, BASE["vocab"], 21)
    taps = []
    O.forward(toks, W, BASE, taps)
    lm.model.residual_tap = got = []
    replay(lm, 20, [([("a", toks)], ["a"])])
    assert len(got) == len(taps)
    for a, b in zip(got, taps):
        close(a, b)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [(2, 2, 2, 20), (7, 3, 2, 14), (1, 24, 1), (13, 13), (20, 2, 2, 2)])
def test_portions(device, cuts):
    lm, W = build(BASE, device)
    toks = tokens(sum(cuts), BASE["vocab"], 3)
    steps, p = [], 0
    for n in cuts:
        steps.append(([("a", toks[p:p + n])], []))
        p += n
    close(replay(lm, 40, steps)["a"], O.forward(toks, W, BASE))


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
        close(got[k], O.forward(seqs[k] + tail[k], W, BASE))


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
    close(got["a"], O.forward(a, W, BASE))
    close(got["c"], O.forward(c, W, BASE))
    close(got["d"], O.forward(d, W, BASE))
    close(got["b"], O.forward(b + [b[0]], W, BASE))


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens_and_long_decoding(device):
    cfg = config([ssm(mlp=dense(16)), attn(mlp=moe()), attn(kv_from=1)], width=32)
    lm, W = build(cfg, device, seed=4)
    toks = tokens(150, cfg["vocab"], 12)
    steps = [([("a", toks[:2])], [])] + [([("a", [t])], []) for t in toks[2:]]
    got = replay(lm, 160, steps)["a"]
    want = O.forward(toks, W, cfg)
    close(got[:8], want[:8])
    close(got, want, 5e-4)


# ------------------------------------------------------------------------- keys far away, made to stand out
FARS = (0, 1, 31, 32, 33, 63, 64, 65, -70)


def _needle_weights(W, cfg, rotated):
    """Layer 0's keys read the leading half of a token's embedding and its queries the other half, and the asking
    token 89+k carries in its query half what the planted token 80+k carries in its key half: the asking token's
    largest score by far is at the planted position, whose value (another token's) differs from its own.
    ``rotated``: part of the match also runs through the rotated, shared key part."""
    m, width = cfg["layers"][0]["mixer"], cfg["width"]
    H, dn, dr, R, qr = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"], m["q_rank"]
    p = "l0.mix."
    for k in range(len(FARS)):
        W["embed"][89 + k, 16:32] = W["embed"][80 + k, :16]
    W[p + "dq"] = torch.zeros(qr, width, dtype=O.F64)
    W[p + "dq"][:, 16:16 + qr] = torch.eye(qr, dtype=O.F64)
    W[p + "dq.norm"] = torch.ones(qr, dtype=O.F64)
    W[p + "dkv"] = torch.cat([torch.eye(R, width, dtype=O.F64), 0.3 * torch.eye(dr, width, dtype=O.F64) * rotated])
    W[p + "dkv.norm"] = torch.ones(R, dtype=O.F64)
    uq = torch.zeros(H, dn + dr, qr, dtype=O.F64)
    uq[:, :dn] = 1.5 * torch.eye(dn, qr, dtype=O.F64)
    if rotated:
        uq[:, dn:] = torch.eye(dr, qr, dtype=O.F64)
    W[p + "uq"] = uq.reshape(H * (dn + dr), qr)
    W[p + "uk"] = torch.eye(dn, R, dtype=O.F64).repeat(H, 1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T,rotated", [(130, False), (130, True), (700, False)])
def test_far_key_stands_out(device, T, rotated):
    """Tokens planted early are asked for at the end: one key far back takes most of the softmax, in a prompt and in
    decoding, at the borders of the 32- and 64-key sweeps and, for the long case, of decode attention's key splits."""
    cfg = config([attn(heads=2, dim=16, rot=8, vdim=8, kv_rank=16, q_rank=16, scale=1.0, base=1e4), attn(kv_from=0, heads=2, dim=16,
                  rot=8, vdim=8, kv_rank=16, q_rank=16, scale=0.5, base=1e4)], width=32, vocab=98, escale=4.0, bigram=(5, 1, 0), alpha=1.0)
    lm, W = build(cfg, device, seed=6, tweak=lambda W: _needle_weights(W, cfg, rotated))
    toks = tokens(T, 80, 13)
    for k, far in enumerate(FARS):
        toks[far % T] = 80 + k                        # planted far back ...
    probe = [89 + k for k in range(len(FARS))]
    full = toks + probe                               # ... and asked for at the end
    want = O.forward(full, W, cfg)
    close(replay(lm, 1100, [([("a", full)], ["a"])])["a"], want)
    steps = [([("a", toks)], [])] + [([("a", [t])], []) for t in probe]
    close(replay(lm, 1100, steps)["a"], want)
    # the planted keys matter: without one the answer differs by far more than the tolerance
    for k in (0, 3, 6, 8):
        other = list(full)
        other[FARS[k] % T] = 5
        i = len(toks) + k
        assert (O.forward(other, W, cfg)[i] - want[i]).abs().max() > 2e-2 * want[i].abs().max()


@pytest.mark.parametrize("device", DEVICES)
def test_state_space_memory_of_far_token(device):
    """A slowly forgetting head keeps what a token wrote hundreds of steps back (prompt in pieces, then decoding)."""
    cfg = config([ssm(heads=2, vdim=8, state=16, groups=1, conv=2, norm_groups=1)], width=32, bigram=None)

    def slow(W):
        W["l0.mix.A_log"] = torch.tensor([-7.0, -6.0], dtype=O.F64)
        W["l0.mix.dt_bias"] = torch.tensor([0.5, 1.0], dtype=O.F64)
    lm, W = build(cfg, device, seed=7, tweak=slow)
    T = 420
    toks = tokens(T, cfg["vocab"], 14)
    want = O.forward(toks, W, cfg)
    steps = [([("a", toks[:17])], []), ([("a", toks[17:400])], [])] + [([("a", [t])], []) for t in toks[400:]]
    close(replay(lm, 500, steps)["a"], want)
    other = list(toks)
    other[3] = (toks[3] + 1) % cfg["vocab"]
    assert (O.forward(other, W, cfg)[-1] - want[-1]).abs().max() > 1e-3 * want[-1].abs().max()


# --------------------------------------------------------------------------------------- other sizes, bf16
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cfg", [
    config([attn(heads=4, dim=16, rot=16, vdim=32, kv_rank=48, q_rank=24, mlp=moe(experts=10, identity=2, top=3, count=3, keep=2))],
           width=64, vocab=130, alpha=1.0),
    config([ssm(heads=8, vdim=16, state=64, groups=4, conv=4, norm_groups=8, mlp=dense(72))], width=40, eps=1e-3),
    config([attn(heads=7, dim=6, rot=2, vdim=10, kv_rank=9, q_rank=5), attn(kv_from=0, heads=1, dim=2, rot=2, vdim=3,
                                                                              kv_rank=9, q_rank=2)], width=24, vocab=31),
])
def test_other_sizes(device, cfg):
    lm, W = build(cfg, device, seed=8)
    toks = tokens(70, cfg["vocab"], 15)
    want = O.forward(toks, W, cfg)
    steps = [([("a", toks[:33])], []), ([("a", toks[33:66])], [])] + [([("a", [t])], []) for t in toks[66:]]
    close(replay(lm, 100, steps)["a"], want)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_weights_and_activations(device):
    """Routed layers take every expert here (top = all outputs), so no choice can flip under bf16 rounding."""
    cfg = config([attn(mlp=dense()), ssm(mlp=moe(experts=3, identity=1, top=4)), attn(kv_from=0, mlp=moe(experts=4, identity=0, top=4))])
    lm, W = build(cfg, device, dtype=torch.bfloat16)
    toks = tokens(40, cfg["vocab"], 17)
    got = replay(lm, 60, [([("a", toks[:30])], [])] + [([("a", [t])], []) for t in toks[30:]])["a"]
    close(got, O.forward(toks, W, cfg), 0.06)


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_matrix_core_sizes_long_context(device):
    """Sizes the matrix-core sweep takes (key rows a multiple of 16, latent a multiple of 32), 300 keys, several key
    splits in decoding."""
    cfg = config([attn(heads=4, dim=32, rot=32, vdim=32, kv_rank=64, q_rank=32, scale=0.15),
                  attn(heads=8, dim=16, rot=32, vdim=16, kv_rank=64, q_rank=32, scale=0.2, kv_from=0)], width=64, vocab=101)
    lm, W = build(cfg, device, seed=12, dtype=torch.bfloat16)
    toks = tokens(300, cfg["vocab"], 19)
    got = replay(lm, 600, [([("a", toks[:290])], [])] + [([("a", [t])], []) for t in toks[290:]])["a"]
    close(got, O.forward(toks, W, cfg), 0.06)


def test_checkpoint_roundtrip_and_registry(tmp_path):
    from safetensors.torch import save_file
    from llm_in_practise_amd.models.registry import load_causal_lm
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in O.random_weights(BASE, 9).items()}
    save_file(W, str(tmp_path / "model.safetensors"))
    (tmp_path / "config.json").write_text(json.dumps(BASE))
    lm = load_causal_lm(str(tmp_path), dtype=torch.float32, device="cpu")
    assert type(lm).__name__ == "DogudraForCausalLM"
    toks = tokens(12, BASE["vocab"], 18)
    close(lm(torch.tensor([toks])).logits[0], O.forward(toks, {k: v.double() for k, v in W.items()}, BASE))
    bad = copy.deepcopy(BASE)
    bad["layers"][0]["type"] = "conv"
    with pytest.raises(ValueError):
        DogudraConfig.from_dict(bad)
    bad = copy.deepcopy(BASE)
    bad["layers"][2]["mixer"]["kv_from"] = 3              # a later layer, and other sizes
    with pytest.raises(ValueError):
        DogudraConfig.from_dict(bad)


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a user starts it: a checkpoint folder, JSON steps on standard input, one file of float
    logits per step that wants any, ``done <step>`` after every step."""
    import os
    import subprocess
    import sys
    import numpy as np
    from safetensors.torch import save_file
    cfg = config([attn(mlp=moe()), ssm(mlp=dense(32)), attn(kv_from=0)], width=40, vocab=53)
    W = {k: v.to(torch.bfloat16).contiguous() for k, v in O.random_weights(cfg, 5).items()}
    model, out = tmp_path / "model", tmp_path / "out"
    model.mkdir()
    save_file(W, str(model / "model.safetensors"))
    (model / "config.json").write_text(json.dumps(cfg))
    a, b = tokens(9, 53, 1), tokens(4, 53, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[7:8], "want": []}, {"id": "b", "tokens": b[3:], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[8:], "want": [0]}], "end": ["a"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, CUDA_VISIBLE_DEVICES="", HIP_VISIBLE_DEVICES="")
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", str(model), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "16"], input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True,
                       text=True, timeout=600, env=env)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    W64 = {k: v.double() for k, v in W.items()}
    wa, wb = O.forward(a, W64, cfg), O.forward(b, W64, cfg)
    got = {n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, 53).copy()) for n in range(3)}
    close(got[0], wa[[0, 6]])
    close(got[1], wb[[3]])
    close(got[2], wa[[8]])


# ------------------------------------------------- greedy generation through the entry points and the scheduler
def _greedy(cfg, W, prompt, n):
    seq = list(prompt)
    for _ in range(n):
        seq.append(int(O.forward(seq, W, cfg)[-1].argmax()))
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
    cfg = config([attn(mlp=moe()), ssm(mlp=dense(32)), attn(kv_from=0)], width=40, vocab=53)
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
    cfg = config([attn(mlp=moe()), ssm(mlp=dense(32)), attn(kv_from=0)], width=40, vocab=53)
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
    close(eager["a"], O.forward(a[:29], W, cfg))
    close(eager["c"], O.forward(c, W, cfg))


@pytest.mark.gpu
def test_expert_paths_agree():
    """The pair-streaming path and the sorted path of the routed experts give the same sums."""
    from llm_in_practise_amd.ops.moe import moe_glu_experts, route_grouped
    g = torch.Generator().manual_seed(3)
    T, Wd, E, F, top = 37, 64, 5, 24, 3
    h = torch.randn(T, Wd, generator=g).cuda()
    wgu, wd = (torch.randn(E, 2, F, Wd, generator=g) / 8).cuda(), (torch.randn(E, Wd, F, generator=g) / 5).cuda()
    idx, w = route_grouped(torch.randn(T, E + 2, generator=g).cuda(), None, top, 1, 1, 1.3)
    sh = torch.randn(T, Wd, generator=g).cuda()
    a = moe_glu_experts(h, wgu, wd, idx, w, 1.0, sh, few_tokens=True)
    b = moe_glu_experts(h, wgu, wd, idx, w, 1.0, sh, few_tokens=False)
    close(a, b.double().cpu(), 1e-5)
    c = moe_glu_experts(h.cpu(), wgu.cpu(), wd.cpu(), idx.cpu(), w.cpu(), 1.0, sh.cpu())
    close(a, c.double(), 1e-5)
