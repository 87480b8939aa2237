"""Plain, slow Vivepel forward pass: the oracle the engine's Vivepel path is tested against.

One function per mechanism, whole sequences only (no cache, no batching, no kernels), written from
the design's equations and sharing no code with `ai_agent_kubectl_amd`.  Everything runs in the dtype
of `x` (tests use float32 or float64); weights are given as a dict name -> tensor with the
checkpoint's names (`embed`, `l<i>.norm1`, `l<i>.mix.q`, ..., `final.norm`, `head`), the
configuration as the parsed config.json dict.

Notation: n tokens, width d; per attention layer H query heads, G key/value heads, head size D.
"""
import math

import torch


def group_rms_norm(x, w, groups, eps):
    """x [n, d] split into `groups` consecutive parts; each part / sqrt(mean(part^2) + eps); times w."""
    n, d = x.shape
    out = torch.empty_like(x)
    step = d // groups
    for g in range(groups):
        part = x[:, g * step:(g + 1) * step]
        out[:, g * step:(g + 1) * step] = part / torch.sqrt((part * part).mean(dim=1, keepdim=True) + eps)
    return out * w.to(x.dtype)


def head_rms_norm(x, w, eps):
    """x [n, heads, D]: every head vector / sqrt(mean^2 + eps), times the shared weight w [D]."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w.to(x.dtype)


def rotary(x, positions, dims, base):
    """x [n, heads, D]; the first `dims` entries of each head are rotated in pairs (i, i + dims/2) by
    the angle position * base^(-2i/dims); the other entries pass through."""
    out = x.clone()
    half = dims // 2
    for t, p in enumerate(positions):
        for i in range(half):
            f = base ** (-2.0 * i / dims)
            a = torch.tensor(float(p), dtype=torch.float32) * torch.tensor(f, dtype=torch.float32)
            c, s = torch.cos(a).to(x.dtype), torch.sin(a).to(x.dtype)
            u, v = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = u * c - v * s
            out[t, :, i + half] = v * c + u * s
    return out


def soft_cap(s, cap):
    return cap * torch.tanh(s / cap)


def chunk_visible(i, j, size):
    """Query position i sees key position j."""
    return j <= i and (i // size) == (j // size)


def sink_softmax_row(scores):
    """Weights of one query over its visible keys, with a sink of score 0 in the denominator."""
    e = torch.exp(scores)
    return e / (1.0 + e.sum())


def attention_mixer(h, W, pre, mc, eps, positions):
    """h [n, d] -> [n, d].  mc: the layer's `mixer` dict of the configuration."""
    n = h.shape[0]
    H, G, D, Dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    dt = h.dtype
    q = h @ W[pre + "q"].to(dt).T + W[pre + "q.b"].to(dt)
    k = h @ W[pre + "k"].to(dt).T + W[pre + "k.b"].to(dt)
    q = q.view(n, H, D)
    k = k.view(n, G, D)
    v = k.clone()                                   # the values are the keys as projected
    q = head_rms_norm(q, W[pre + "q.norm"], eps)
    k = head_rms_norm(k, W[pre + "k.norm"], eps)
    q = rotary(q, positions, mc["rot"]["dims"], mc["rot"]["base"])
    k = rotary(k, positions, mc["rot"]["dims"], mc["rot"]["base"])
    size = mc["mask"]["size"]
    talk = W[pre + "talk"].to(dt)
    rep = H // G
    out = torch.zeros(n, H, Dv, dtype=dt)
    for t in range(n):
        i = positions[t]
        vis = [u for u in range(n) if chunk_visible(i, positions[u], size)]
        weights = torch.zeros(H, len(vis), dtype=dt)
        for g in range(H):
            s = torch.stack([(q[t, g] * k[u, g // rep]).sum() for u in vis]) * mc["scale"]
            weights[g] = sink_softmax_row(soft_cap(s, mc["softcap"]))
        mixed = talk @ weights                      # [H, keys]: head a takes sum_g talk[a, g] weights[g]
        for a in range(H):
            for c, u in enumerate(vis):
                out[t, a] += mixed[a, c] * v[u, a // rep]
    return out.reshape(n, H * Dv) @ W[pre + "o"].to(dt).T


def poly_norm(z, coef, eps):
    """coef = (a, b, c, e): a N(z) + b N(z^2) + c N(z^3) + e, N = divide the row by its rms."""
    def N(y):
        return y / torch.sqrt((y * y).mean(dim=1, keepdim=True) + eps)
    a, b, c, e = [float(t) for t in coef]
    return a * N(z) + b * N(z * z) + c * N(z * z * z) + e


def feed_forward(h, W, pre, eps):
    z = h @ W[pre + "up"].to(h.dtype).T
    return poly_norm(z, W[pre + "act"].float(), eps) @ W[pre + "down"].to(h.dtype).T


def forward(config, W, tokens, dtype=torch.float32, positions=None):
    """-> (logits [n, vocab], residual stream after every layer [layers, n, d])."""
    eps, groups = config["norm"]["eps"], config["norm"]["groups"]
    positions = list(range(len(tokens))) if positions is None else positions
    x = W["embed"].to(dtype)[torch.tensor(tokens)]
    trail = []
    for li, layer in enumerate(config["layers"]):
        p = "l%d." % li
        assert layer["type"] == "attention"
        y = attention_mixer(group_rms_norm(x, W[p + "norm1"], groups, eps), W, p + "mix.", layer["mixer"], eps,
                            positions)
        x = x + W[p + "ls1"].to(dtype) * group_rms_norm(y, W[p + "norm1b"], groups, eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            y = feed_forward(group_rms_norm(x, W[p + "norm2"], groups, eps), W, p + "mlp.", eps)
            x = x + W[p + "ls2"].to(dtype) * group_rms_norm(y, W[p + "norm2b"], groups, eps)
        trail.append(x.clone())
    logits = group_rms_norm(x, W["final.norm"], groups, eps) @ W["head"].to(dtype).T
    return logits, torch.stack(trail)


def random_config(gen, layers=2, width=64, vocab=96, groups=2, **over):
    """A small configuration dict in the checkpoint's layout; `over` replaces mixer / mlp entries."""
    out = {"architecture": "Vivepel", "vocab": vocab, "width": width, "norm": {"eps": 1e-5, "groups": groups},
           "layers": []}
    for _ in range(layers):
        mixer = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "mask": {"size": 8},
                 "rot": {"base": 1000.0, "dims": 8}, "scale": 0.25, "softcap": 20.0}
        mixer.update({k: v for k, v in over.items() if k in mixer})
        mlp = {"kind": "dense", "ff": over.get("ff", 48)} if over.get("mlp", True) else None
        out["layers"].append({"type": "attention", "mixer": mixer, "mlp": mlp})
    return out


def random_weights(config, seed=0, dtype=torch.bfloat16, std=None):
    """Random weights with the checkpoint's names and shapes for `config`."""
    g = torch.Generator().manual_seed(seed)
    d, V = config["width"], config["vocab"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else (std or i ** -0.5))).to(dtype)

    def vec(n, lo=0.5, hi=1.5):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    W = {"embed": mat(V, d, 1.0), "head": mat(V, d), "final.norm": vec(d)}
    for li, layer in enumerate(config["layers"]):
        p, m = "l%d." % li, layer["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        for nm in ("norm1", "norm1b"):
            W[p + nm] = vec(d)
        W[p + "ls1"] = vec(d, 0.2, 1.0)
        W[p + "mix.q"], W[p + "mix.q.b"] = mat(H * D, d), (torch.randn(H * D, generator=g) * 0.3).to(dtype)
        W[p + "mix.k"], W[p + "mix.k.b"] = mat(G * D, d), (torch.randn(G * D, generator=g) * 0.3).to(dtype)
        W[p + "mix.q.norm"], W[p + "mix.k.norm"] = vec(D), vec(D)
        W[p + "mix.talk"] = (torch.eye(H) * 0.7 + torch.randn(H, H, generator=g) * 0.3).to(dtype)
        W[p + "mix.o"] = mat(d, H * Dv)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            for nm in ("norm2", "norm2b"):
                W[p + nm] = vec(d)
            W[p + "ls2"] = vec(d, 0.2, 1.0)
            W[p + "mlp.up"], W[p + "mlp.down"] = mat(ff, d), mat(d, ff)
            W[p + "mlp.act"] = torch.tensor([0.6, 0.3, 0.2, 0.05]).to(dtype) + (torch.randn(4, generator=g) * 0.05).to(dtype)
    return W
