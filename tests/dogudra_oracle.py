"""Plain, slow Dogudra: one function per mechanism, token by token, float64 on the CPU.

The yardstick of the Dogudra tests.  It shares nothing with the product path (``models/dogudra.py``, the ops under
``llm_in_practise_amd/ops`` and the HIP kernels): no packed batches, no slots, no cache object, no absorbed
projections — every function takes one sequence ``[tokens, features]`` and loops where the mechanism is causal or
recurrent.  Keys and values of the latent attention are expanded per head here, exactly as the definition reads.

``W`` is a dict name -> float64 tensor with the checkpoint's own names (``l2.mix.uk`` ...), ``cfg`` the parsed
``config.json`` dict.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def norm_centered(x, w, eps):
    """Weight stored as an offset from one."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def embed(tokens, W, cfg):
    """Token row times the scale plus a hashed row for the (previous, current) pair; the first token of a sequence
    takes the table's extra last row."""
    e = cfg["embedding"]
    x = W["embed"][tokens] * float(e["scale"])
    bg = e.get("bigram")
    if bg:
        n = int(bg["buckets"])
        for t, tok in enumerate(tokens):
            row = n if t == 0 else (int(tokens[t - 1]) * int(bg["mul_prev"]) + int(tok) * int(bg["mul_cur"])) % n
            x[t] = x[t] + W["bigram"][row]
    return x


def rotate_pairs(v, positions, dims, base):
    """v [T, ..., d]: neighbours (2i, 2i+1) of the first ``dims`` entries turn by position * base^(-2i/dims)."""
    out = v.clone()
    for r, p in enumerate(positions):
        for i in range(dims // 2):
            a = p * base ** (-2.0 * i / dims)
            c, s = math.cos(a), math.sin(a)
            u, w = v[r, ..., 2 * i].clone(), v[r, ..., 2 * i + 1].clone()
            out[r, ..., 2 * i] = u * c - w * s
            out[r, ..., 2 * i + 1] = w * c + u * s
    return out


def latent_kv(h, W, p, m, eps):
    """What a layer with its own down-projection caches: the normed latent and the rotated shared key part."""
    T = h.shape[0]
    r, dr = int(m["kv_rank"]), int(m["rot_dim"])
    d = h @ W[p + "dkv"].T
    c = norm_plain(d[:, :r], W[p + "dkv.norm"], eps)
    kr = rotate_pairs(d[:, r:r + dr], range(T), int(m["rot"]["dims"]), float(m["rot"]["base"]))
    return c, kr


def latent_attention(h, W, p, m, eps, c, kr):
    """h [T, width]; c [T, kv_rank] and kr [T, rot_dim] are this layer's own or the ones of the layer it borrows."""
    T = h.shape[0]
    H, dn, dr, dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    cq = norm_plain(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, dn + dr)
    qn = q[..., :dn]
    qr = rotate_pairs(q[..., dn:], range(T), int(m["rot"]["dims"]), float(m["rot"]["base"]))
    kn = (c @ W[p + "uk"].T).view(T, H, dn)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    gate = torch.sigmoid(h @ W[p + "g"].T)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        for i in range(T):
            s = (kn[: i + 1, hd] @ qn[i, hd] + kr[: i + 1] @ qr[i, hd]) * float(m["scale"])
            out[i, hd] = torch.softmax(s, 0) @ v[: i + 1, hd]
        out[:, hd] = out[:, hd] * gate[:, hd:hd + 1]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def causal_conv(u, w, b):
    """u [T, C], w [C, taps] (last column: the current token), b [C]; zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        y[t] = b
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] = y[t] + w[:, j] * u[s]
    return y


def mamba2_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * P
    silu = torch.nn.functional.silu
    zxbcdt = h @ W[p + "in"].T
    z = zxbcdt[:, :inner]
    xbc = silu(causal_conv(zxbcdt[:, inner:2 * inner + 2 * G * N], W[p + "conv"], W[p + "conv.b"]))
    dt = torch.nn.functional.softplus(zxbcdt[:, 2 * inner + 2 * G * N:] + W[p + "dt_bias"])
    x = xbc[:, :inner].view(T, H, P)
    Bm = xbc[:, inner:inner + G * N].view(T, G, N)
    Cm = xbc[:, inner + G * N:].view(T, G, N)
    y = torch.zeros(T, H, P, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=h.dtype)
        rate = math.exp(float(W[p + "A_log"][hd]))
        for t in range(T):
            S = math.exp(-rate * float(dt[t, hd])) * S + float(dt[t, hd]) * torch.outer(Bm[t, g], x[t, hd])
            y[t, hd] = S.T @ Cm[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = int(m["norm_groups"])
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def dense_ff(h, W, p):
    return gelu_tanh(h @ W[p + "up"].T) @ W[p + "down"].T


def clipped_expert(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def route(h, W, p, r):
    """Per token: the chosen expert indices and their weights."""
    E, idn, top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
    n = E + idn
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + W[p + "correction"] if p + "correction" in W else s.clone()
    gr = r.get("groups")
    picks = []
    for t in range(h.shape[0]):
        c = choice[t].clone()
        if gr and int(gr["count"]) > 1:
            cnt, keep = int(gr["count"]), int(gr["keep"])
            size = n // cnt
            best = sorted(range(cnt), key=lambda g: (-float(c[g * size:(g + 1) * size].max()), g))[:keep]
            for g in range(cnt):
                if g not in best:
                    c[g * size:(g + 1) * size] = -math.inf
        order = sorted(range(n), key=lambda e: (-float(c[e]), e))[:top]
        picks.append([(e, float(s[t, e]) * float(r["scale"])) for e in order])
    return picks


def moe_ff(h, W, p, mlp):
    r = mlp["router"]
    E = int(r["experts"])
    out = torch.zeros_like(h)
    for t, chosen in enumerate(route(h, W, p, r)):
        for e, w in chosen:
            if e >= E:
                out[t] = out[t] + w * h[t]
            else:
                out[t] = out[t] + w * clipped_expert(h[t:t + 1], W, f"{p}e{e}.", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        out = out + clipped_expert(h, W, p + "shared.", float(mlp["shared"]["limit"]))
    return out


def forward(tokens, W, cfg, taps=None):
    """Logits [T, vocab] of one sequence from its first token; ``taps`` (a list) receives the stream after every
    layer."""
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    x = embed(list(tokens), W, cfg)
    held = {}
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", lc["mixer"]
        if lc["type"] == "mamba2":
            y = mamba2_mixer(x, W, p, m, eps)
        elif lc["type"] == "latent_attention":
            if m.get("kv_from") is None:
                held[i] = latent_kv(x, W, p, m, eps)
            c, kr = held[i if m.get("kv_from") is None else int(m["kv_from"])]
            y = latent_attention(x, W, p, m, eps, c, kr)
        else:
            raise ValueError(lc["type"])
        x = norm_centered(alpha * x + y, W[f"l{i}.norm1"], eps)
        mlp = lc.get("mlp")
        if mlp is not None:
            y = dense_ff(x, W, f"l{i}.mlp.") if mlp["kind"] == "dense" else moe_ff(x, W, f"l{i}.mlp.", mlp)
            x = norm_centered(alpha * x + y, W[f"l{i}.norm2"], eps)
        if taps is not None:
            taps.append(x.clone())
    return norm_centered(x, W["final.norm"], eps) @ W["head"].T


def checkpoint_shapes(cfg):
    """Names and shapes of the tensors a config asks for (the test's own list, from the layer descriptions)."""
    Wd, V = int(cfg["width"]), int(cfg["vocab"])
    out = [("embed", (V, Wd)), ("final.norm", (Wd,)), ("head", (V, Wd))]
    bg = cfg["embedding"].get("bigram")
    if bg:
        out.append(("bigram", (int(bg["buckets"]) + 1, Wd)))
    for i, lc in enumerate(cfg["layers"]):
        m, p = lc["mixer"], f"l{i}.mix."
        out.append((f"l{i}.norm1", (Wd,)))
        if lc["type"] == "latent_attention":
            H, dn, dr, dv, R, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out += [(p + "dq", (qr, Wd)), (p + "dq.norm", (qr,)), (p + "uq", (H * (dn + dr), qr)), (p + "uk", (H * dn, R)),
                    (p + "uv", (H * dv, R)), (p + "g", (H, Wd)), (p + "o", (Wd, H * dv))]
            if m.get("kv_from") is None:
                out += [(p + "dkv", (R + dr, Wd)), (p + "dkv.norm", (R,))]
        else:
            H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            ch = H * P + 2 * G * N
            out += [(p + "in", (2 * H * P + 2 * G * N + H, Wd)), (p + "conv", (ch, taps)), (p + "conv.b", (ch,)),
                    (p + "dt_bias", (H,)), (p + "A_log", (H,)), (p + "D", (H,)), (p + "norm", (H * P,)), (p + "o", (Wd, H * P))]
        mlp, p = lc.get("mlp"), f"l{i}.mlp."
        if mlp is None:
            continue
        out.append((f"l{i}.norm2", (Wd,)))
        if mlp["kind"] == "dense":
            out += [(p + "up", (mlp["ff"], Wd)), (p + "down", (Wd, mlp["ff"]))]
        else:
            r, F = mlp["router"], mlp["expert"]["ff"]
            n = r["experts"] + r.get("identity", 0)
            out += [(p + "router", (n, Wd)), (p + "correction", (n,))]
            for e in range(r["experts"]):
                out += [(f"{p}e{e}.gate", (F, Wd)), (f"{p}e{e}.up", (F, Wd)), (f"{p}e{e}.down", (Wd, F))]
            if mlp.get("shared"):
                Fs = mlp["shared"]["ff"]
                out += [(p + "shared.gate", (Fs, Wd)), (p + "shared.up", (Fs, Wd)), (p + "shared.down", (Wd, Fs))]
    return out


def random_weights(cfg, seed=0):
    """float64 weights: matrices ~ N(0, 1/in) (router and gates a little stronger, so choices are not near ties),
    norm offsets and corrections small, step-size biases and decay rates in a stable range."""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in checkpoint_shapes(cfg):
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith("mix.conv"):
            t = torch.randn(shape, generator=g, dtype=F64) * 0.5
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g, dtype=F64) / math.sqrt(shape[1])
            if leaf in ("embed", "bigram"):
                t = t * math.sqrt(shape[1]) * 0.6
            if leaf == "router":
                t = t * 3.0
        elif name.endswith(("dq.norm", "dkv.norm", "mix.norm")):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g, dtype=F64)
        elif leaf == "dt_bias":
            t = torch.rand(shape, generator=g, dtype=F64) * 3.0 - 2.5
        elif leaf == "A_log":
            t = torch.rand(shape, generator=g, dtype=F64) * 2.0 - 1.0
        elif leaf == "D":
            t = 1.0 + 0.3 * torch.randn(shape, generator=g, dtype=F64)
        elif leaf == "correction":
            t = 0.1 * torch.randn(shape, generator=g, dtype=F64)
        else:
            t = 0.2 * torch.randn(shape, generator=g, dtype=F64)
        W[name] = t
    return W
