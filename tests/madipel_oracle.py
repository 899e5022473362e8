"""Plain, slow Madipel in fp64 on the CPU: one function per mechanism, written from the design's equations.

Shares nothing with the product path.  ``cfg`` is a config.json-style dict, ``W`` maps checkpoint tensor names to
tensors.  Notation: i = query position, j = key position, H query heads over G key/value heads.
"""
import math

import torch

F64 = torch.float64


def sin_positions(positions, width):
    """s[p, 2i] = sin(p * 10000^(-2i/width)), s[p, 2i+1] = cos(same)."""
    out = torch.zeros(len(positions), width, dtype=F64)
    for r, p in enumerate(positions):
        for c in range(width):
            i = c // 2
            a = p * (10000.0 ** (-2.0 * i / width))
            out[r, c] = math.sin(a) if c % 2 == 0 else math.cos(a)
    return out


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms_norm_whole(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the whole projection row (all heads together)."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def xielu(z, p, q):
    sp = math.log1p(math.exp(p))
    sq = math.log1p(math.exp(q))
    pos = sp * z * z + z / 2
    neg = (0.5 + sq) * (torch.exp(torch.clamp(z, max=0.0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def window_attention(q, k, v, H, G, window, scale, temp, r1, r2):
    """q [n, H, D], k [n, G, D], v [n, G, Dv] of ONE sequence (positions 0..n-1) -> [n, H*Dv].
    score = q.k * scale * temp_h - r1_h ln(1 + r2_h (i - j)), visible iff 0 <= i - j < window."""
    n, Dv = q.shape[0], v.shape[-1]
    out = torch.zeros(n, H, Dv, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(n):
            lo = max(0, i - window + 1)
            dist = torch.arange(i - lo, -1, -1, dtype=F64)  # i - j for j = lo .. i
            s = (k[lo:i + 1, g] @ q[i, h]) * scale * temp[h] - r1[h] * torch.log(1 + r2[h] * dist)
            p = torch.softmax(s, 0)
            out[i, h] = (p[:, None] * v[lo:i + 1, g]).sum(0)
    return out.reshape(n, H * Dv)


def forward(cfg, W, tokens, layers_out=None):
    """Logits [n, vocab] (fp64) of one sequence given whole."""
    W = {k: t.to(F64) for k, t in W.items()}
    n, d, eps = len(tokens), cfg["width"], cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] + sin_positions(list(range(n)), d)
    v_first = None
    for li, L in enumerate(cfg["layers"]):
        p, m = f"l{li}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        h = layer_norm(x, W[p + "norm1"], W[p + "norm1.b"], eps)
        q = rms_norm_whole(h @ W[p + "mix.q"].T, W[p + "mix.q.norm"], eps)
        k = rms_norm_whole(h @ W[p + "mix.k"].T, W[p + "mix.k.norm"], eps)
        v = h @ W[p + "mix.v"].T
        if m.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                lam = float(W[p + "mix.vmix"])
                v = (1 - lam) * v + lam * v_first
        a = window_attention(q.view(n, H, D), k.view(n, G, D), v.view(n, G, Dv), H, G, m["mask"]["size"], m["scale"],
                             W[p + "mix.temp"], W[p + "mix.r1"], W[p + "mix.r2"])
        y = a @ W[p + "mix.o"].T
        if L.get("mlp") is not None:
            pq = W[p + "mlp.act"]
            y = y + xielu(h @ W[p + "mlp.up"].T, float(pq[0]), float(pq[1])) @ W[p + "mlp.down"].T
        x = x + cfg["residual_mult"] * y
        if layers_out is not None:
            layers_out.append(x.clone())
    y = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return (y @ W["head"].T) * cfg["logit_scale"]


# ------------------------------------------------------------------ small models for the tests
def make_config(width, vocab, layers, eps=1e-5, residual_mult=0.4, logit_scale=0.5):
    """``layers``: dicts with heads, kv_heads, dim, vdim, window, scale, v_mix, ff (None: no feed-forward)."""
    out = []
    for L in layers:
        out.append({"type": "attention",
                    "mixer": {"heads": L["heads"], "kv_heads": L["kv_heads"], "dim": L["dim"], "vdim": L["vdim"],
                              "mask": {"size": L["window"]}, "scale": L.get("scale", 1.0 / math.sqrt(L["dim"])),
                              "v_mix": L.get("v_mix", False)},
                    "mlp": None if L.get("ff") is None else {"kind": "dense", "ff": L["ff"]}})
    return {"architecture": "Madipel", "layers": out, "logit_scale": logit_scale, "norm": {"eps": eps},
            "residual_mult": residual_mult, "vocab": vocab, "width": width}


def make_weights(cfg, seed):
    """Random bf16-representable weights under the checkpoint's tensor names."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    W = {"embed": rnd(V, d), "final.norm": (1 + rnd(d, s=0.1).float()).to(torch.bfloat16), "final.norm.b": rnd(d, s=0.05),
         "head": rnd(V, d, s=d ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}."
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = (1 + rnd(d, s=0.1).float()).to(torch.bfloat16)
        W[p + "norm1.b"] = rnd(d, s=0.05)
        W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = rnd(H * D, d, s=d ** -0.5), rnd(G * D, d, s=d ** -0.5), rnd(G * Dv, d, s=d ** -0.5)
        W[p + "mix.q.norm"] = (1 + rnd(H * D, s=0.2).float()).to(torch.bfloat16)
        W[p + "mix.k.norm"] = (1 + rnd(G * D, s=0.2).float()).to(torch.bfloat16)
        W[p + "mix.vmix"] = (torch.rand((), generator=g) * 0.6 + 0.1).to(torch.bfloat16)
        W[p + "mix.r1"] = (torch.rand(H, generator=g) + 0.2).to(torch.bfloat16)
        W[p + "mix.r2"] = (torch.rand(H, generator=g) + 0.2).to(torch.bfloat16)
        W[p + "mix.temp"] = (torch.rand(H, generator=g) * 2 + 1.0).to(torch.bfloat16)
        W[p + "mix.o"] = rnd(d, H * Dv, s=(H * Dv) ** -0.5)
        if L["mlp"] is not None:
            ff = L["mlp"]["ff"]
            W[p + "mlp.up"], W[p + "mlp.down"] = rnd(ff, d, s=d ** -0.5), rnd(d, ff, s=ff ** -0.5)
            W[p + "mlp.act"] = rnd(2, s=0.7)
    return W
