"""Plain float64 oracle of the Levovik design: whole sequences, no cache, no batching, one function
per mechanism, every loop written out.  Shares no code with the product path.

A model is (config dict, weights dict name -> tensor).  ``forward`` returns the logits of every
position of one sequence and, optionally, the residual stream after every layer.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def scaled_frequencies(rot: dict) -> torch.Tensor:
    """dims/2 rotation frequencies base^(-2i/dims), long wavelengths slowed down by ``scaling``
    {factor, low, high, original}: wavelengths under original/high keep their frequency, those over
    original/low get frequency/factor, and between the two the frequency is blended linearly in
    original/wavelength."""
    dims = int(rot["dims"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if sc:
            fac, lo, hi, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            lam = 2.0 * math.pi / f
            if lam < orig / hi:
                pass
            elif lam > orig / lo:
                f = f / fac
            else:
                s = (orig / lam - lo) / (hi - lo)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate(x, pos: int, freq, interleaved: bool):
    """x [heads, dim]: the first 2 len(freq) entries of every head turn by pos * freq."""
    n = freq.numel()
    y = x.clone()
    for i in range(n):
        a, b = (2 * i, 2 * i + 1) if interleaved else (i, i + n)
        ang = pos * freq[i]
        c, s = torch.cos(ang), torch.sin(ang)
        y[:, a] = x[:, a] * c - x[:, b] * s
        y[:, b] = x[:, b] * c + x[:, a] * s
    return y


def softmax_attention(q, k, v, scale: float, sink=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H*dv]; causal over the whole prefix.
    ``sink`` [H]: one more term exp(sink[h]) in every denominator, with no value."""
    T, H, _ = q.shape
    G, dv = k.shape[1], v.shape[2]
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            s = (k[: i + 1, g] @ q[i, h]) * scale
            m = s.max()
            if sink is not None:
                m = torch.maximum(m, sink[h])
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e / den) @ v[: i + 1, g]
    return out.reshape(T, H * dv)


def attention_a(h, w: dict, pre: str, m: dict, eps: float):
    """The left mixer of a ``parallel`` layer: rotation (half layout) first, then q and k divided by
    their root mean square per head (no weight), learned sinks."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + "q"].T).view(T, H, dk)
    k = (h @ w[pre + "k"].T).view(T, G, dk)
    v = (h @ w[pre + "v"].T).view(T, G, dv)
    fr = scaled_frequencies(m["rot"])
    q = torch.stack([rms(rotate(q[t], t, fr, False), eps) for t in range(T)])
    k = torch.stack([rms(rotate(k[t], t, fr, False), eps) for t in range(T)])
    o = softmax_attention(q, k, v, float(m["scale"]), sink=w[pre + "sink"])
    return o @ w[pre + "o"].T


def attention_b(h, w: dict, pre: str, m: dict, eps: float):
    """The left mixer of a ``parallel_2`` layer: weighted RMS norm of q and k per head, then rotation
    (interleaved layout); the values are the keys as projected; ordinary softmax."""
    T = h.shape[0]
    H, G, dk = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (h @ w[pre + "q"].T).view(T, H, dk)
    k = (h @ w[pre + "k"].T).view(T, G, dk)
    v = k.clone()
    fr = scaled_frequencies(m["rot"])
    q = torch.stack([rotate(rms(q[t], eps) * w[pre + "q.norm"], t, fr, True) for t in range(T)])
    k = torch.stack([rotate(rms(k[t], eps) * w[pre + "k.norm"], t, fr, True) for t in range(T)])
    o = softmax_attention(q, k, v, float(m["scale"]))
    return o @ w[pre + "o"].T


def causal_conv_silu(x, cw):
    """x [T, C], cw [C, taps] (last column: the current token); zeros before the start."""
    T, C = x.shape
    taps = cw.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1 - j)
            if s >= 0:
                y[t] += cw[:, j] * x[s]
    return silu(y)


def gated_delta(h, w: dict, pre: str, m: dict, eps: float):
    """The right mixer of a ``parallel`` layer: the delta rule with a decay per head and key channel."""
    T = h.shape[0]
    H, Gk, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = causal_conv_silu(h @ w[pre + "q"].T, w[pre + "q.conv"]).view(T, Gk, dk)
    k = causal_conv_silu(h @ w[pre + "k"].T, w[pre + "k.conv"]).view(T, Gk, dk)
    v = causal_conv_silu(h @ w[pre + "v"].T, w[pre + "v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)  # [T, H]
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]
    dec = torch.exp(-torch.exp(w[pre + "A_log"]).view(1, H, 1) * softplus(z).view(T, H, dk))
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // Gk)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = dec[t, hh].view(dk, 1) * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, hh] = S.T @ q[t, g]
    out = rms(out, eps) * w[pre + "norm"] * gate
    return out.reshape(T, H * dv) @ w[pre + "o"].T


def gated_linear(h, w: dict, pre: str, m: dict, eps: float):
    """The right mixer of a ``parallel_2`` layer: linear attention with a decay per key channel."""
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ w[pre + "k"].T).view(T, H, dk)
    v = (h @ w[pre + "v"].T).view(T, H, dv)
    z = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / float(m["tau"]))).view(T, H, dk)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = alpha[t, hh].view(dk, 1) * S + torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = S.T @ q[t, hh]
    out = rms(out, eps) * w[pre + "norm"]
    return (out.reshape(T, H * dv) * silu(h @ w[pre + "g"].T)) @ w[pre + "o"].T


def dense_ff(h, w: dict, pre: str):
    return (torch.relu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def route(h, w: dict, pre: str, r: dict):
    """(experts [T, top], weights [T, top]): sigmoid scores; experts in ``count`` equal neighbouring
    groups, a group scored by the sum of its two largest; only the ``keep`` best groups stay."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(h @ w[pre + "router"].T)
    T = s.shape[0]
    ids = torch.zeros(T, top, dtype=torch.long)
    wt = torch.zeros(T, top, dtype=F64)
    gr = r.get("groups")
    for t in range(T):
        ok = [True] * E
        if gr:
            cnt, keep = int(gr["count"]), int(gr["keep"])
            per = E // cnt
            gs = []
            for g in range(cnt):
                part = sorted(s[t, g * per:(g + 1) * per].tolist(), reverse=True)
                gs.append(sum(part[:2]))
            best = sorted(range(cnt), key=lambda g: -gs[g])[:keep]
            ok = [(e // per) in best for e in range(E)]
        cand = sorted([e for e in range(E) if ok[e]], key=lambda e: -float(s[t, e]))[:top]
        ids[t] = torch.tensor(cand)
        sc = s[t, cand]
        wt[t] = sc / (sc.sum() + 1e-20) * float(r["scale"])
    return ids, wt


def expert(h, w: dict, pre: str, limit: float):
    g = torch.clamp(h @ w[pre + "gate"].T, max=limit)
    u = torch.clamp(h @ w[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[pre + "down"].T


def moe_ff(h, w: dict, pre: str, ml: dict):
    ids, wt = route(h, w, pre, ml["router"])
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            out[t] += wt[t, j] * expert(h[t:t + 1], w, f"{pre}e{e}.", float(ml["expert"]["limit"]))[0]
    return out


def side_input(x, tokens, i: int, w: dict, side_dim: int, eps: float):
    """The per-layer token input of layer i, to be added to the stream x [T, d]."""
    e = w["side.embed"][tokens][:, i * side_dim:(i + 1) * side_dim]
    g = gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e
    y = g @ w[f"l{i}.side.proj"].T
    return rms(y, eps) * w[f"l{i}.side.norm"]


def forward(cfg: dict, weights: dict, tokens, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of one sequence."""
    w = {k: v.to(F64) if v.is_floating_point() else v for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tok] * float((cfg.get("embedding") or {}).get("scale", 1.0))
    side = cfg.get("token_side")
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = L["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        if L["type"] == "parallel":
            a = attention_a(h, w, p + "mix.left.", m["left"], eps)
            b = gated_delta(h, w, p + "mix.right.", m["right"], eps)
        elif L["type"] == "parallel_2":
            a = attention_b(h, w, p + "mix.left.", m["left"], eps)
            b = gated_linear(h, w, p + "mix.right.", m["right"], eps)
        else:
            raise ValueError(L["type"])
        x = x + float(m["left_scale"]) * a + float(m["right_scale"]) * b
        ml = L.get("mlp")
        if ml is not None:
            h2 = layer_norm(x, w[p + "norm2"], eps)
            x = x + (dense_ff(h2, w, p + "mlp.") if ml["kind"] == "dense" else moe_ff(h2, w, p + "mlp.", ml))
        if side:
            x = x + side_input(x, tok, i, w, int(side["dim"]), eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    hf = layer_norm(x, w["final.norm"], eps)
    return (hf @ w["head"].T) * float(cfg.get("logit_scale", 1.0))


def layers_of(cfg: dict, weights: dict, tokens) -> torch.Tensor:
    """The residual stream after every layer, [layers, T, width]."""
    out: list = []
    forward(cfg, weights, tokens, layers_out=out)
    return torch.stack(out)


def greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    """``n`` tokens by repeated whole-sequence forwards, each the argmax of the last logits."""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(forward(cfg, w, seq)[-1]))
        out.append(t)
        seq.append(t)
    return out


def random_weights(cfg: dict, seed: int = 0) -> dict:
    """Random tensors of a config's shapes (values a bf16 checkpoint could hold), by name.  The inner
    sizes of the two-stage projections are the mixer's ``a_rank`` / ``g_rank`` (absent: 5 and 7)."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    w = {"embed": rnd(V, d, std=0.8 / float((cfg.get("embedding") or {}).get("scale", 1.0))),
         "final.norm": rnd(d, std=0.1, mean=1.0), "head": rnd(V, d, std=2 * d ** -0.5)}
    sd = int((cfg.get("token_side") or {}).get("dim", 0))
    if sd:
        w["side.embed"] = rnd(V, sd * len(cfg["layers"]), std=0.8)
    for i, spec in enumerate(cfg["layers"]):
        L, m = f"l{i}.", spec["mixer"]
        w[L + "norm1"] = rnd(d, std=0.1, mean=1.0)
        a, b, P, Q = m["left"], m["right"], f"l{i}.mix.left.", f"l{i}.mix.right."
        H, G, dk = a["heads"], a["kv_heads"], a["dim"]
        w[P + "q"], w[P + "k"] = rnd(H * dk, d, std=1.5 * d ** -0.5), rnd(G * dk, d, std=1.5 * d ** -0.5)
        if spec["type"] == "parallel":
            dv = a["vdim"]
            w[P + "v"], w[P + "sink"] = rnd(G * dv, d, std=d ** -0.5), rnd(H, std=1.0)
        else:
            dv = dk
            w[P + "q.norm"], w[P + "k.norm"] = rnd(dk, std=0.2, mean=1.0), rnd(dk, std=0.2, mean=1.0)
        w[P + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        H, dk, dv = b["heads"], b["dim"], b["vdim"]
        ra, rg = int(b.get("a_rank", 5)), int(b.get("g_rank", 7))
        if spec["type"] == "parallel":
            Gk, taps = b["kv_heads"], b["conv"]
            for n, rows in (("q", Gk * dk), ("k", Gk * dk), ("v", H * dv)):
                w[Q + n], w[Q + n + ".conv"] = rnd(rows, d, std=1.5 * d ** -0.5), rnd(rows, taps, std=0.5)
            w[Q + "b"] = rnd(H, d, std=2 * d ** -0.5)
            w[Q + "A_log"], w[Q + "dt_bias"] = rnd(H, std=0.6, mean=-0.5), rnd(H * dk, std=0.7, mean=-1.0)
            w[Q + "a1"], w[Q + "a2"] = rnd(ra, d, std=d ** -0.5), rnd(H * dk, ra, std=2 * ra ** -0.5)
            w[Q + "g1"], w[Q + "g2"] = rnd(rg, d, std=d ** -0.5), rnd(H * dv, rg, std=2 * rg ** -0.5)
        else:
            for n, rows in (("q", H * dk), ("k", H * dk), ("v", H * dv), ("g", H * dv)):
                w[Q + n] = rnd(rows, d, std=1.2 * d ** -0.5)
            w[Q + "a1"], w[Q + "a2"] = rnd(ra, d, std=d ** -0.5), rnd(H * dk, ra, std=2 * ra ** -0.5)
            w[Q + "a2.b"] = rnd(H * dk, std=1.0, mean=2.0)
        w[Q + "norm"] = rnd(dv, std=0.1, mean=1.0)
        w[Q + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        ml = spec.get("mlp")
        if ml is not None:
            w[L + "norm2"] = rnd(d, std=0.1, mean=1.0)
            if ml["kind"] == "dense":
                f = ml["ff"]
                w[L + "mlp.gate"], w[L + "mlp.up"] = rnd(f, d, std=d ** -0.5), rnd(f, d, std=d ** -0.5)
                w[L + "mlp.down"] = rnd(d, f, std=f ** -0.5)
            else:
                f = ml["expert"]["ff"]
                for e in range(ml["router"]["experts"]):
                    # pre-activations on both sides of the limit
                    w[f"{L}mlp.e{e}.gate"], w[f"{L}mlp.e{e}.up"] = rnd(f, d, std=1.5 * d ** -0.5), rnd(f, d, std=1.5 * d ** -0.5)
                    w[f"{L}mlp.e{e}.down"] = rnd(d, f, std=f ** -0.5)
                w[L + "mlp.router"] = rnd(ml["router"]["experts"], d, std=2 * d ** -0.5)
        if sd:
            w[L + "side.gate"], w[L + "side.proj"] = rnd(sd, d, std=d ** -0.5), rnd(d, sd, std=sd ** -0.5)
            w[L + "side.norm"] = rnd(d, std=0.1, mean=0.5)
    return w
