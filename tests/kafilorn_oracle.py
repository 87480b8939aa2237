"""Plain per-token implementation of the Kafilorn decoder, written from its equations; shares no code with
the package.  One function per mechanism.  Everything is computed in one floating type (`DT`, float64 by
default) on the checkpoint's own tensor names, for one sequence at a time and without any cache: every
call recomputes the whole sequence.

Notation: h is a sublayer's input row, W x means `W @ x` with W stored [out, in].
"""
from __future__ import annotations

import math

import torch

DT = torch.float64


def f(t):
    return t.to(DT)


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, var = mean of squared deviations; no bias."""
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * f(w)


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rotate(x, pos, base, dims):
    """Rotary position on the first `dims` entries of the last axis; entry i pairs with i + dims/2."""
    half = dims // 2
    if half == 0:
        return x
    i = torch.arange(half, dtype=DT)
    ang = float(pos) * (float(base) ** (-2.0 * i / dims))
    c, s = torch.cos(ang), torch.sin(ang)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def mlstm(hs, T, p, m, eps):
    """hs [n, width] -> [n, width].  Matrix memory with exponential gating and a running maximum."""
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    cap = m.get("gate_cap")
    S = torch.zeros(H, D, Dv, dtype=DT)
    nrm = torch.zeros(H, D, dtype=DT)
    mx = torch.zeros(H, dtype=DT)
    out = []
    for h in hs:
        q = (f(T[p + "q"]) @ h).view(H, D) * D ** -0.5
        k = (f(T[p + "k"]) @ h).view(H, D)
        v = (f(T[p + "v"]) @ h).view(H, Dv)
        ig = f(T[p + "i"]) @ h + f(T[p + "i.b"])
        fg = f(T[p + "f"]) @ h + f(T[p + "f.b"])
        if cap:
            ig = cap * torch.tanh(ig / cap)
            fg = cap * torch.tanh(fg / cap)
        fg = torch.nn.functional.logsigmoid(fg)
        m_new = torch.maximum(fg + mx, ig)
        a, b = torch.exp(fg + mx - m_new), torch.exp(ig - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[:, :, None] * v[:, None, :]
        nrm = a[:, None] * nrm + b[:, None] * k
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q)
        den = torch.maximum((nrm * q).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        o = rms_div(num / den[:, None], eps).reshape(-1) * f(T[p + "norm"])
        o = o * torch.sigmoid(f(T[p + "g"]) @ h)
        out.append(f(T[p + "o"]) @ o)
    return torch.stack(out)


def latent_kv(hs, T, p, m, eps):
    """The cached part of a latent-attention layer: (c [n, kv_rank] normed, shared rotated key part [n, rot_dim])."""
    R, Dr = m["kv_rank"], m["rot_dim"]
    rot = m.get("rot")
    cs, ks = [], []
    for pos, h in enumerate(hs):
        d = f(T[p + "dkv"]) @ h
        cs.append(rms_div(d[:R], eps) * f(T[p + "dkv.norm"]))
        ks.append(rotate(d[R:], pos, rot["base"], rot["dims"]) if rot else d[R:])
    return torch.stack(cs), torch.stack(ks)


def latent_attention(hs, T, p, m, eps, kv):
    """hs [n, width] -> [n, width]; kv = (c, k_rot) of this layer or of the layer it borrows them from."""
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot, mask = m.get("rot"), m.get("mask")
    c, kr = kv
    kn = (c @ f(T[p + "uk"]).T).view(-1, H, D)           # unrotated keys  [n, H, D]
    vv = (c @ f(T[p + "uv"]).T).view(-1, H, Dv)          # values          [n, H, Dv]
    sink = f(T[p + "sink"]) if (p + "sink") in T else None
    out = []
    for i, h in enumerate(hs):
        cq = rms_div(f(T[p + "dq"]) @ h, eps) * f(T[p + "dq.norm"])
        q = (f(T[p + "uq"]) @ cq).view(H, D + Dr)
        qn, qr = q[:, :D], q[:, D:]
        if rot:
            qr = rotate(qr, i, rot["base"], rot["dims"])
        lo = max(0, i - mask["size"] + 1) if mask else 0
        s = (torch.einsum("hd,jhd->hj", qn, kn[lo:i + 1]) + qr @ kr[lo:i + 1].T) * m["scale"]
        mxs = s.max(-1, keepdim=True).values
        if sink is not None:
            mxs = torch.maximum(mxs, sink[:, None])
        e = torch.exp(s - mxs)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[:, None] - mxs)
        o = torch.einsum("hj,jhv->hv", e / den, vv[lo:i + 1]).reshape(-1)
        out.append(f(T[p + "o"]) @ o)
    return torch.stack(out)


def dense_ff(h, T, p):
    return f(T[p + "down"]) @ torch.relu(f(T[p + "up"]) @ h) ** 2


def gated_expert(h, T, p):
    return f(T[p + "down"]) @ (torch.nn.functional.silu(f(T[p + "gate"]) @ h) * (f(T[p + "up"]) @ h))


def route(h, T, p, r):
    """-> (chosen expert ids, their weights) for one row."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(f(T[p + "router"]) @ h, -1)
    choice = s + f(T[p + "correction"]) if (p + "correction") in T else s.clone()
    g = r.get("groups")
    if g:
        per = E // g["count"]
        best = choice.view(g["count"], per).max(-1).values
        keep = torch.topk(best, g["keep"]).indices
        allowed = torch.zeros(g["count"], dtype=torch.bool)
        allowed[keep] = True
        choice = torch.where(allowed.repeat_interleave(per), choice, torch.full_like(choice, -math.inf))
    ids = torch.topk(choice, top).indices
    w = s[ids]
    return ids, w / (w.sum() + 1e-20)


def moe_ff(h, T, p, mlp):
    ids, w = route(h, T, p, mlp["router"])
    y = sum(wi * gated_expert(h, T, f"{p}e{int(e)}.") for e, wi in zip(ids, w))
    if mlp.get("shared"):
        y = y + gated_expert(h, T, p + "shared.")
    return y


def feed_forward(hs, T, p, mlp):
    if mlp["kind"] == "dense":
        return torch.stack([dense_ff(h, T, p) for h in hs])
    if mlp["kind"] == "moe":
        return torch.stack([moe_ff(h, T, p, mlp) for h in hs])
    raise ValueError(mlp["kind"])


def forward(cfg, T, tokens, layer_out=None):
    """tokens (one sequence) -> logits [n, vocab]; layer_out(i, x [n, width]) after every layer (streams summed)."""
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    x0 = f(T["embed"])[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    xs = [x0.clone() for _ in range(S)] if S else [x0]
    kvs = {}
    for li, L in enumerate(cfg["layers"]):
        lp = f"l{li}."
        for q in (1, 2):
            if q == 2 and L.get("mlp") is None:
                continue
            hc = f"{lp}hc{q}."
            u = sum(f(T[hc + "in"])[s] * xs[s] for s in range(S)) if S else xs[0]
            hs = layer_norm(u, T[f"{lp}norm{q}"], eps)
            if q == 2:
                y = feed_forward(hs, T, lp + "mlp.", L["mlp"])
            elif L["type"] == "mlstm":
                y = mlstm(hs, T, lp + "mix.", L["mixer"], eps)
            elif L["type"] == "latent_attention":
                m = L["mixer"]
                src = m.get("kv_from")
                if src is None:
                    kvs[li] = latent_kv(hs, T, lp + "mix.", m, eps)
                    src = li
                y = latent_attention(hs, T, lp + "mix.", m, eps, kvs[src])
            else:
                raise ValueError(L["type"])
            if S:
                mix, o = f(T[hc + "mix"]), f(T[hc + "out"])
                xs = [sum(mix[s, t] * xs[s] for s in range(S)) + o[t] * y for t in range(S)]
            else:
                xs = [xs[0] + y]
        if layer_out is not None:
            layer_out(li, sum(xs))
    x = layer_norm(sum(xs), T["final.norm"], eps)
    return x @ f(T["head"]).T * cfg.get("logit_scale", 1.0)


# ---------------------------------------------------------------------------------------------------
# small random models for the tests (their own sizes; nothing here comes from the package)
def mlstm_layer(heads=2, dim=8, vdim=8, gate_cap=15.0, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim}
    if gate_cap:
        m["gate_cap"] = gate_cap
    return {"type": "mlstm", "mixer": m, "mlp": mlp}


def attention_layer(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=12, kv_rank=16, window=8, base=100.0, scale=None, kv_from=None,
                    mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot_dim:
        m["rot"] = {"base": base, "dims": rot_dim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=16, groups=(3, 2), shared=16):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    d = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def make_config(layers, width=32, vocab=96, streams=2, embed_scale=4.0, logit_scale=0.5, eps=1e-6):
    c = {"architecture": "Kafilorn", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
         "logit_scale": logit_scale, "layers": layers}
    if streams:
        c["streams"] = streams
    return c


def random_tensors(cfg, seed=0, dtype=torch.bfloat16):
    """Random checkpoint tensors for `cfg` (bf16-representable values, as a checkpoint stores them)."""
    g = torch.Generator().manual_seed(seed)
    h, V, S = cfg["width"], cfg["vocab"], cfg.get("streams")

    def mat(o, i, std=None):
        return (torch.randn(o, i, generator=g) * (std if std is not None else i ** -0.5)).to(dtype)

    def vec(n, lo=0.7, hi=1.3):
        return (lo + (hi - lo) * torch.rand(n, generator=g)).to(dtype)

    T = {"embed": mat(V, h, 1.0), "head": mat(V, h), "final.norm": vec(h)}
    for i, L in enumerate(cfg["layers"]):
        c, m, f = f"l{i}.", L["mixer"], L.get("mlp")
        for q in ("1", "2") if f is not None else ("1",):
            T[c + "norm" + q] = vec(h)
            if S:
                T[c + f"hc{q}.in"] = vec(S, 0.4 / S, 1.6 / S)
                T[c + f"hc{q}.out"] = vec(S, 0.4, 1.1)
                T[c + f"hc{q}.mix"] = (torch.eye(S) * 0.7 + torch.rand(S, S, generator=g) * (0.4 / S)).to(dtype)
        if L["type"] == "mlstm":
            H = m["heads"]
            for k, n in (("q", m["dim"]), ("k", m["dim"]), ("v", m["vdim"]), ("g", m["vdim"])):
                T[c + "mix." + k] = mat(H * n, h)
            T[c + "mix.i"], T[c + "mix.f"] = mat(H, h, 2.0 * h ** -0.5), mat(H, h, 2.0 * h ** -0.5)
            T[c + "mix.i.b"] = torch.randn(H, generator=g).to(dtype)
            T[c + "mix.f.b"] = (2.0 + torch.randn(H, generator=g)).to(dtype)
            T[c + "mix.norm"], T[c + "mix.o"] = vec(H * m["vdim"]), mat(h, H * m["vdim"])
        else:
            H = m["heads"]
            T[c + "mix.dq"], T[c + "mix.dq.norm"] = mat(m["q_rank"], h), vec(m["q_rank"])
            T[c + "mix.uq"] = mat(H * (m["dim"] + m["rot_dim"]), m["q_rank"], 2.0 * m["q_rank"] ** -0.5)
            if m.get("kv_from") is None:
                T[c + "mix.dkv"], T[c + "mix.dkv.norm"] = mat(m["kv_rank"] + m["rot_dim"], h), vec(m["kv_rank"])
            T[c + "mix.uk"] = mat(H * m["dim"], m["kv_rank"], 2.0 * m["kv_rank"] ** -0.5)
            T[c + "mix.uv"] = mat(H * m["vdim"], m["kv_rank"])
            T[c + "mix.sink"] = torch.randn(H, generator=g).to(dtype)
            T[c + "mix.o"] = mat(h, H * m["vdim"])
        if f is None:
            continue
        if f["kind"] == "dense":
            T[c + "mlp.up"], T[c + "mlp.down"] = mat(f["ff"], h), mat(h, f["ff"])
        else:
            E = f["router"]["experts"]
            T[c + "mlp.router"] = mat(E, h, 3.0 * h ** -0.5)
            T[c + "mlp.correction"] = (torch.randn(E, generator=g) * (0.6 / E)).to(dtype)
            names = [f"mlp.e{e}." for e in range(E)] + (["mlp.shared."] if f.get("shared") else [])
            for n in names:
                ff = f["shared"]["ff"] if n == "mlp.shared." else f["expert"]["ff"]
                T[c + n + "gate"], T[c + n + "up"], T[c + n + "down"] = mat(ff, h), mat(ff, h), mat(h, ff)
    return T
