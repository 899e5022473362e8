"""Plain, slow Merudra in fp64 on the CPU: one function per mechanism, written from the design's equations.

Shares nothing with the product path.  ``cfg`` is a config.json-style dict, ``W`` maps checkpoint tensor names to
tensors.  Notation: t = time step (position), H heads over G key heads, D key size, Dv value size, d model width.
"""
import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def causal_conv(x, w):
    """y_t = sum_j w[:, j] x_(t - taps + 1 + j); x [n, c], w [c, taps]; zeros before t = 0."""
    n, taps = x.shape[0], w.shape[1]
    y = torch.zeros_like(x)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return y


def input_conv(h, w):
    """What a sublayer reads: h + conv(h)."""
    return h + causal_conv(h, w)


def query_temperature(positions, coef, every):
    return torch.tensor([1 + coef * math.log((p + 1) // every + 1) for p in positions], dtype=F64)


def softmax_attention(q, k, v, H, G, scale):
    """q [n, H, D], k [n, G, D], v [n, G, Dv] of one sequence from position 0 -> [n, H*Dv]; causal."""
    n, Dv = q.shape[0], v.shape[-1]
    out = torch.zeros(n, H, Dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(n):
            s = (k[:i + 1, g] @ q[i, h]) * scale
            p = torch.softmax(s, 0)
            out[i, h] = (p[:, None] * v[:i + 1, g]).sum(0)
    return out.reshape(n, H * Dv)


def attention_mixer(h, W, p, m, eps, positions=None):
    """The 'attention' mixer on input h [n, d]; p = '<layer>.mix.'; m = the layer's mixer config."""
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(n, H, D)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(n, G, D)
    v = k.clone()                       # the values are the keys as projected
    assert Dv == D
    pos = list(range(n)) if positions is None else positions
    qn = rms_unit(q, eps) * query_temperature(pos, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None, None]
    kn = rms_unit(k, eps)
    a = softmax_attention(qn, kn, v, H, G, m["scale"])
    a = a * torch.sigmoid(h @ W[p + "g"].T)
    return a @ W[p + "o"].T


def delta_rule(q, k, v, beta, g, S=None):
    """Gated delta rule of one head.  q, k [n, D]; v [n, Dv]; beta, g [n].  Returns (o [n, Dv], S [D, Dv])."""
    n, D, Dv = q.shape[0], q.shape[1], v.shape[1]
    S = torch.zeros(D, Dv, dtype=F64) if S is None else S.clone()
    o = torch.zeros(n, Dv, dtype=F64)
    for t in range(n):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def delta_mixer(h, W, p, m, eps):
    n = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(n, G, D)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(n, G, D)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(n, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    gate = silu(h @ W[p + "g"].T).view(n, H, Dv)
    out = torch.zeros(n, H, Dv, dtype=F64)
    for hh in range(H):
        kv = hh // (H // G)
        o, _ = delta_rule(q[:, kv], k[:, kv], v[:, hh], beta[:, hh], g[:, hh])
        out[:, hh] = rms_unit(o, eps) * W[p + "norm"] * gate[:, hh]
    return out.reshape(n, H * Dv) @ W[p + "o"].T


def route(h, W, p, r):
    """Router: (chosen ids [n, top], weights [n, top]); ids >= experts are identity experts."""
    s = torch.softmax(h @ W[p + "router"].T, -1)
    ids = torch.topk(s + W[p + "correction"], r["top"], dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def moe(h, W, p, mlp):
    r = mlp["router"]
    ids, wt = route(h, W, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), wt[t]):
            if e >= r["experts"]:
                out[t] += w * h[t]
            else:
                pe = f"{p}e{e}."
                out[t] += w * ((silu(h[t] @ W[pe + "gate"].T) * (h[t] @ W[pe + "up"].T)) @ W[pe + "down"].T)
    return out


def token_side(x, tokens, W, p, li, dim, eps):
    e = W["side.embed"][torch.tensor(tokens)][:, li * dim:(li + 1) * dim]
    y = (gelu_tanh(x @ W[p + "side.gate"].T) * e) @ W[p + "side.proj"].T
    return rms_unit(y, eps) * W[p + "side.norm"]


def forward(cfg, W, tokens, layers_out=None):
    """Logits [n, vocab] (fp64) of one sequence given whole."""
    W = {k: t.to(F64) for k, t in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    X = [x]
    for li, L in enumerate(cfg["layers"]):
        p = f"l{li}."
        h = input_conv(x, W[p + "canon1"])
        y = attention_mixer(h, W, p + "mix.", L["mixer"], eps) if L["type"] == "attention" else \
            delta_mixer(h, W, p + "mix.", L["mixer"], eps)
        y = y * torch.sigmoid(x @ W[p + "rg1"].T + W[p + "rg1.b"])
        x = x + rms_unit(y, eps) * W[p + "norm1"]
        if L.get("mlp"):
            h = input_conv(x, W[p + "canon2"])
            y = moe(h, W, p + "mlp.", L["mlp"]) * torch.sigmoid(x @ W[p + "rg2"].T + W[p + "rg2.b"])
            x = x + rms_unit(y, eps) * W[p + "norm2"]
        x = x + token_side(x, tokens, W, p, li, cfg["token_side"]["dim"], eps)
        X.append(x)
        x = sum(W[p + "dwa"][j] * X[j] for j in range(li + 2))
        if layers_out is not None:
            layers_out.append(x)
    return (rms_unit(x, eps) * W["final.norm"]) @ W["head"].T


# ------------------------------------------------------------------ test models
def make_config(width, vocab, layers, taps=3, side=5, eps=1e-5):
    """config.json of a small model.  ``layers``: dicts with type, heads, kv_heads, dim, vdim and, for attention,
    scale / coef / every; for delta, conv; ``mlp``: None or dict(experts, identity, top, ff)."""
    out = []
    for L in layers:
        if L["type"] == "attention":
            mixer = {"heads": L["heads"], "kv_heads": L["kv_heads"], "dim": L["dim"], "vdim": L["dim"], "scale": L.get("scale", 0.3),
                     "q_temp": {"coef": L.get("coef", 0.4), "every": L.get("every", 7)}}
        else:
            mixer = {"heads": L["heads"], "kv_heads": L["kv_heads"], "dim": L["dim"], "vdim": L["vdim"], "conv": L.get("conv", 4)}
        m = L.get("mlp")
        mlp = None if m is None else {"kind": "moe", "expert": {"ff": m["ff"]},
                                      "router": {"experts": m["experts"], "identity": m["identity"], "top": m["top"]}}
        out.append({"type": L["type"], "mixer": mixer, "mlp": mlp})
    return {"architecture": "Merudra", "canon": {"taps": taps}, "layers": out, "norm": {"eps": eps},
            "token_side": {"dim": side}, "vocab": vocab, "width": width}


def make_weights(cfg, seed):
    """Random bf16 tensors under the checkpoint's names; scales chosen so that every mechanism matters."""
    g = torch.Generator().manual_seed(seed)
    d, V, taps, sd = cfg["width"], cfg["vocab"], cfg["canon"]["taps"], cfg["token_side"]["dim"]

    def rn(*shape, s=1.0):
        return torch.randn(*shape, generator=g) * s

    def lin(o, i):
        return rn(o, i, s=i ** -0.5)

    W = {"embed": rn(V, d), "side.embed": rn(V, sd * len(cfg["layers"])), "final.norm": 1 + rn(d, s=0.1), "head": lin(V, d)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W.update({p + "norm1": 1 + rn(d, s=0.1), p + "canon1": rn(d, taps, s=0.3), p + "rg1": lin(d, d), p + "rg1.b": rn(d, s=0.3),
                  p + "dwa": rn(i + 2, s=0.3), p + "side.gate": lin(sd, d), p + "side.proj": lin(d, sd), p + "side.norm": 1 + rn(d, s=0.1)})
        W[p + "dwa"][-1] += 1.0
        if L["type"] == "attention":
            W.update({p + "mix.q": lin(H * D, d), p + "mix.q.b": rn(H * D, s=0.2), p + "mix.k": lin(G * D, d),
                      p + "mix.k.b": rn(G * D, s=0.2), p + "mix.g": lin(H * Dv, d), p + "mix.o": lin(d, H * Dv)})
        else:
            c = m["conv"]
            W.update({p + "mix.q": lin(G * D, d), p + "mix.q.conv": rn(G * D, c, s=0.6), p + "mix.k": lin(G * D, d),
                      p + "mix.k.conv": rn(G * D, c, s=0.6), p + "mix.v": lin(H * Dv, d), p + "mix.v.conv": rn(H * Dv, c, s=0.6),
                      p + "mix.b": lin(H, d), p + "mix.a": lin(H, d), p + "mix.A_log": rn(H, s=0.7), p + "mix.dt_bias": rn(H),
                      p + "mix.norm": 1 + rn(Dv, s=0.1), p + "mix.g": lin(H * Dv, d), p + "mix.o": lin(d, H * Dv)})
        if L["mlp"] is not None:
            r, ff = L["mlp"]["router"], L["mlp"]["expert"]["ff"]
            ne = r["experts"] + r["identity"]
            W.update({p + "norm2": 1 + rn(d, s=0.1), p + "canon2": rn(d, taps, s=0.3), p + "rg2": lin(d, d), p + "rg2.b": rn(d, s=0.3),
                      p + "mlp.router": lin(ne, d) * 2, p + "mlp.correction": rn(ne, s=0.15)})
            for e in range(r["experts"]):
                W.update({f"{p}mlp.e{e}.gate": lin(ff, d), f"{p}mlp.e{e}.up": lin(ff, d), f"{p}mlp.e{e}.down": lin(d, ff)})
    return {k: v.to(torch.bfloat16) for k, v in W.items()}
