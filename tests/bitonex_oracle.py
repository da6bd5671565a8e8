"""Plain float64 oracle of the Bitonex design: one function per mechanism, whole sequences at once,
no cache, no batching, nothing shared with the product path.

A model is (config dict in the ``config.json`` dialect, {tensor name: tensor}).  ``forward`` returns
the logits of every position and the residual stream after every layer.

Notation.  ``x`` [n, width] is the residual stream of one sequence, positions 0 .. n-1.
``rms(v) = v / sqrt(mean(v^2) + eps)``.

* block:      x <- x + m * mixer(h) * sigmoid(R1 h + b1),  h = g1 * rms(x)      (g1 one number)
              x <- x + m * ff(h2)   * sigmoid(R2 h2 + b2), h2 = g2 * rms(x)     (if the layer has a ff)
* attention:  grouped-query softmax attention, causal; the first ``rot.dims`` entries of every q / k
              head turn by position (entry i pairs with i + dims/2); score = q.k * scale * temp[head];
              heads * sigmoid(G h) -> O
* lightning:  q, k, v = silu(projections); per head S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t;
              rms over all heads' outputs together * weight, * sigmoid(G h) -> O
* latent:     c_q = w_q * rms(Dq h), q = Uq c_q, per head [dim plain | rot_dim turning];
              Dkv h = [kv_rank | rot_dim]: c = w_c * rms(first part), second part turns (shared by all
              heads; entries 2i, 2i+1 pair); per head k = [Uk c | shared], v = Uv c; softmax, causal -> O;
              ``kv_from`` j: c and the shared part are layer j's
* ff:         Down (gelu_tanh(Gate h) * Up h)
* output:     logits = cap * tanh(Head (g_f * rms(x)) / cap)
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * sigmoid(z)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def angles(n: int, dims: int, base: float, start: int = 0) -> torch.Tensor:
    """[n, dims / 2]: position * base^(-2 i / dims)."""
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.tensor(base, dtype=F64) ** (-2.0 * i / dims)
    return torch.arange(start, start + n, dtype=F64)[:, None] * f[None, :]


def turn_half(v: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v [n, heads, size]: entry i (< dims/2) pairs with entry i + dims/2; entries from dims on pass."""
    a = angles(v.shape[0], dims, base)[:, None, :]
    c, s = torch.cos(a), torch.sin(a)
    h = dims // 2
    u, w = v[..., :h], v[..., h:dims]
    return torch.cat([u * c - w * s, w * c + u * s, v[..., dims:]], -1)


def turn_pairs(v: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v [n, heads, size]: entry 2i pairs with entry 2i + 1 (i < dims/2); entries from dims on pass."""
    a = angles(v.shape[0], dims, base)[:, None, :]
    c, s = torch.cos(a), torch.sin(a)
    u, w = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = u * c - w * s
    out[..., 1:dims:2] = w * c + u * s
    return out


def causal_softmax(scores: torch.Tensor) -> torch.Tensor:
    """scores [heads, n, n] (query, key): weights over keys j <= i."""
    n = scores.shape[-1]
    keep = torch.tril(torch.ones(n, n, dtype=torch.bool))
    s = scores.masked_fill(~keep, -math.inf)
    s = s - s.max(-1, keepdim=True).values
    e = torch.exp(s)
    return e / e.sum(-1, keepdim=True)


def attention(h: torch.Tensor, w: dict, m: dict) -> torch.Tensor:
    n = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, dk)
    k = (h @ w["k"].T).view(n, G, dk)
    v = (h @ w["v"].T).view(n, G, dv)
    q = turn_half(q, m["rot"]["dims"], m["rot"]["base"])
    k = turn_half(k, m["rot"]["dims"], m["rot"]["base"])
    per = H // G
    out = torch.empty(n, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // per
        sc = (q[:, hd] @ k[:, g].T) * m["scale"] * w["temp"][hd]
        out[:, hd] = causal_softmax(sc[None])[0] @ v[:, g]
    gate = sigmoid(h @ w["g"].T)
    return (out.reshape(n, H * dv) * gate) @ w["o"].T


def lightning(h: torch.Tensor, w: dict, m: dict, eps: float) -> torch.Tensor:
    n = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(n, H, dk)
    k = silu(h @ w["k"].T).view(n, H, dk)
    v = silu(h @ w["v"].T).view(n, H, dv)
    out = torch.empty(n, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(n):
            S = m["decay"][hd] * S + torch.outer(k[t, hd], v[t, hd])
            out[t, hd] = S.T @ q[t, hd]
    y = rms(out.reshape(n, H * dv), eps) * w["norm"]
    return (y * sigmoid(h @ w["g"].T)) @ w["o"].T


def latent_kv(h: torch.Tensor, w: dict, m: dict, eps: float) -> tuple:
    """(c [n, kv_rank], shared turning key part [n, rot_dim]) of a layer with a projection of its own."""
    R, dr = m["kv_rank"], m["rot_dim"]
    d = h @ w["dkv"].T
    c = rms(d[:, :R], eps) * w["dkv.norm"]
    kr = turn_pairs(d[:, None, R:R + dr], m["rot"]["dims"], m["rot"]["base"])[:, 0]
    return c, kr


def latent_attention(h: torch.Tensor, w: dict, m: dict, eps: float, kv: tuple) -> torch.Tensor:
    n = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c, kr = kv
    cq = rms(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(n, H, dn + dr)
    qn = q[..., :dn]
    qr = turn_pairs(q[..., dn:], m["rot"]["dims"], m["rot"]["base"])
    kn = (c @ w["uk"].T).view(n, H, dn)
    v = (c @ w["uv"].T).view(n, H, dv)
    out = torch.empty(n, H, dv, dtype=F64)
    for hd in range(H):
        sc = (qn[:, hd] @ kn[:, hd].T + qr[:, hd] @ kr.T) * m["scale"]
        out[:, hd] = causal_softmax(sc[None])[0] @ v[:, hd]
    return out.reshape(n, H * dv) @ w["o"].T


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    return (gelu_tanh(h @ w["gate"].T) * (h @ w["up"].T)) @ w["down"].T


def _sub(tensors: dict, prefix: str) -> dict:
    return {k[len(prefix):]: v.to(F64) for k, v in tensors.items() if k.startswith(prefix)}


def forward(cfg: dict, tensors: dict, tokens: list, return_layers: bool = False):
    """Logits [n, vocab] in float64 (``return_layers``: and the residual stream after every layer,
    [layers, n, width])."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    t = {k: v.to(F64) for k, v in tensors.items()}
    x = t["embed"][torch.tensor(tokens, dtype=torch.long)]
    kept: dict = {}
    after = []
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        m, w = spec["mixer"], _sub(tensors, p + "mix.")
        h = rms(x, eps) * t[p + "norm1"]
        if spec["type"] == "attention":
            y = attention(h, w, m)
        elif spec["type"] == "lightning":
            y = lightning(h, w, m, eps)
        elif spec["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = latent_kv(h, w, m, eps)
            y = latent_attention(h, w, m, eps, kept[i if src is None else src])
        else:
            raise ValueError(spec["type"])
        x = x + mult * y * sigmoid(h @ t[p + "rg1"].T + t[p + "rg1.b"])
        if spec.get("mlp") is not None:
            h2 = rms(x, eps) * t[p + "norm2"]
            x = x + mult * dense_ff(h2, _sub(tensors, p + "mlp.")) * sigmoid(h2 @ t[p + "rg2"].T + t[p + "rg2.b"])
        after.append(x.clone())
    z = (rms(x, eps) * t["final.norm"]) @ t["head"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap > 0:
        z = cap * torch.tanh(z / cap)
    return (z, torch.stack(after)) if return_layers else z


def random_weights(cfg: dict, seed: int = 0) -> dict:
    """Random tensors of a config's shapes (values a bf16 checkpoint could hold), by name."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def one(mean=1.0):
        return rnd(1, std=0.15, mean=mean).reshape(())

    w = {"embed": rnd(V, d, std=0.8), "final.norm": one(), "head": rnd(V, d, std=2 * d ** -0.5)}
    for i, spec in enumerate(cfg["layers"]):
        L, m, P = f"l{i}.", spec["mixer"], f"l{i}.mix."
        w[L + "norm1"] = one()
        w[L + "rg1"], w[L + "rg1.b"] = rnd(d, d, std=d ** -0.5), rnd(d, std=0.7)
        H = m["heads"]
        if spec["type"] == "attention":
            G, dk, dv = m["kv_heads"], m["dim"], m["vdim"]
            w[P + "q"], w[P + "k"] = rnd(H * dk, d, std=1.5 * d ** -0.5), rnd(G * dk, d, std=1.5 * d ** -0.5)
            w[P + "v"], w[P + "g"] = rnd(G * dv, d, std=d ** -0.5), rnd(H * dv, d, std=d ** -0.5)
            w[P + "temp"] = rnd(H, std=0.4, mean=1.2)
            w[P + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        elif spec["type"] == "lightning":
            dk, dv = m["dim"], m["vdim"]
            w[P + "q"], w[P + "k"] = rnd(H * dk, d, std=d ** -0.5), rnd(H * dk, d, std=d ** -0.5)
            w[P + "v"], w[P + "g"] = rnd(H * dv, d, std=d ** -0.5), rnd(H * dv, d, std=d ** -0.5)
            w[P + "norm"] = rnd(H * dv, std=0.1, mean=1.0)
            w[P + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        else:
            dn, dr, dv, R, Q = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[P + "dq"], w[P + "dq.norm"] = rnd(Q, d, std=d ** -0.5), rnd(Q, std=0.1, mean=1.0)
            w[P + "uq"] = rnd(H * (dn + dr), Q, std=1.5 * Q ** -0.5)
            if m.get("kv_from") is None:
                w[P + "dkv"], w[P + "dkv.norm"] = rnd(R + dr, d, std=d ** -0.5), rnd(R, std=0.1, mean=1.0)
            w[P + "uk"] = rnd(H * dn, R, std=1.5 * R ** -0.5)
            w[P + "uv"] = rnd(H * dv, R, std=R ** -0.5)
            w[P + "o"] = rnd(d, H * dv, std=(H * dv) ** -0.5)
        ml = spec.get("mlp")
        if ml is None:
            continue
        f = ml["ff"]
        w[L + "norm2"] = one()
        w[L + "rg2"], w[L + "rg2.b"] = rnd(d, d, std=d ** -0.5), rnd(d, std=0.7)
        w[L + "mlp.gate"], w[L + "mlp.up"] = rnd(f, d, std=1.5 * d ** -0.5), rnd(f, d, std=d ** -0.5)
        w[L + "mlp.down"] = rnd(d, f, std=f ** -0.5)
    return w


def greedy(cfg: dict, w: dict, prompt, n: int) -> list:
    """``n`` tokens by repeated whole-sequence forwards, each the argmax of the last logits."""
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(torch.argmax(forward(cfg, w, seq)[-1]))
        out.append(t)
        seq.append(t)
    return out
