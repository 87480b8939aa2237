"""Kafilorn in the engine against the plain oracle (tests/kafilorn_oracle.py).

Every test makes its own small configuration and random (or crafted) weights, writes them as a checkpoint
folder (config.json + model.safetensors: the reader and the loader are under test too), builds the engine on it
and compares logits with the oracle's whole-sequence forward.  The same bodies run on the CPU (the ops' torch
references) and, marked `gpu`, on the HIP kernels in fp32 and bf16.
"""
import json
import os

import numpy as np
import pytest
import torch

import kafilorn_oracle as oracle
from kafilorn_oracle import attention_layer, dense, make_config, mlstm_layer, moe

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def write_checkpoint(path, config, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def session(path, device, dtype="float32", max_tokens=256, max_requests=4):
    from ai_agent_kubectl_amd.engine.trace import TraceSession

    return TraceSession(path, dtype=dtype, max_tokens=max_tokens, device=device, max_requests=max_requests)


def replay(sess, tokens, cuts, rid="r", end=True):
    """Feed `tokens` in portions of the sizes `cuts`; logits of every position [n, vocab]."""
    out, at = [], 0
    for c in cuts:
        part = tokens[at:at + c]
        last = at + c >= len(tokens)
        out.append(sess.step([{"id": rid, "tokens": part, "want": list(range(len(part)))}], [rid] if last and end else []))
        at += c
    assert at == len(tokens)
    return np.concatenate(out)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float(np.sqrt((d ** 2).mean(-1)).max() / np.sqrt((w ** 2).mean()))


def row_errs(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean())


def bf16_close(got, want):
    """bf16 rounding can turn a close router call: most rows within the bf16 tolerance, the typical row well within."""
    e = row_errs(got, want)
    return np.median(e) < tol("bfloat16") / 3 and np.mean(e < tol("bfloat16")) >= 0.85


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def tokens_for(config, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def want_logits(config, W, tokens):
    return oracle.forward(config, W, tokens).numpy()


def variant(name):
    if name == "base":            # every kind of layer once; window 8 is half a page
        return make_config([mlstm_layer(mlp=dense(40)), attention_layer(mlp=moe()), attention_layer(kv_from=1, mlp=dense(24)),
                            mlstm_layer(heads=1, dim=12, vdim=20, mlp=moe(experts=4, top=1, groups=None, shared=0))])
    if name == "attention_first":  # attention before any recurrence, three streams, odd sizes, window 21 over a page border
        return make_config([attention_layer(heads=3, dim=10, rot_dim=6, vdim=7, q_rank=9, kv_rank=22, window=21, mlp=dense(33)),
                            mlstm_layer(heads=3, dim=5, vdim=9, gate_cap=4.0),
                            attention_layer(heads=5, dim=4, rot_dim=6, vdim=6, q_rank=11, kv_rank=22, window=3, kv_from=0,
                                            mlp=moe(experts=8, top=3, ff=12, groups=(4, 2), shared=20))],
                           width=36, vocab=80, streams=3, embed_scale=1.0, logit_scale=2.0)
    if name == "plain_residual":   # no streams entry: the plain pre-norm residual; no window; uncapped gates; no mlp
        return make_config([mlstm_layer(heads=2, dim=16, vdim=8, gate_cap=None), attention_layer(window=0, mlp=None),
                            attention_layer(heads=1, dim=16, vdim=16, kv_from=1, window=1, mlp=dense(16))],
                           width=24, vocab=72, streams=None)
    if name == "one_stream":       # one hyper-connected stream (weights that are not 1), every expert chosen
        return make_config([attention_layer(mlp=moe(experts=2, top=2, groups=(1, 1), shared=8)), mlstm_layer(mlp=dense(8))],
                           width=16, vocab=64, streams=1)
    raise KeyError(name)


VARIANTS = ["base", "attention_first", "plain_residual", "one_stream"]


def model_for(tmp_path, name, seed=0):
    c = variant(name)
    W = oracle.random_tensors(c, seed)
    return c, W, write_checkpoint(tmp_path / name, c, W)


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: ops.mixers (torch reference on CPU, HIP kernel on GPU) against the oracle
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S,width", [(1, 24), (2, 64), (4, 100), (7, 256)])
def test_streams_norm_and_update(device, S, width):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(S)
    x = torch.randn(5, S, width, generator=g) * 3 + 2          # a mean far from 0: an RMS norm would differ
    y = torch.randn(5, width, generator=g)
    w_in, out, w_next = torch.rand(S, generator=g), torch.rand(S, generator=g), torch.rand(S, generator=g)
    mix = torch.rand(S, S, generator=g)
    w, w2 = torch.rand(width, generator=g) + 0.5, torch.rand(width, generator=g) + 0.5
    u = sum(w_in[s] * x[:, s] for s in range(S)).double()
    want_h = oracle.layer_norm(u, w, 1e-5)
    got_h = mixers.stream_norm(x.to(device), w_in.to(device), w.to(device), 1e-5, torch.float32)
    assert torch.allclose(got_h.cpu().double(), want_h, rtol=1e-4, atol=1e-4)
    assert not torch.allclose(oracle.rms_div(u, 1e-5) * w, want_h, rtol=1e-2, atol=1e-2)
    new = torch.stack([sum(mix[s, r] * x[:, s] for s in range(S)) + out[r] * y for r in range(S)], dim=1)
    xd = x.clone().to(device)
    for nxt in (False, True):
        xd = x.clone().to(device)
        h2 = mixers.stream_update(xd, y.to(device), mix.to(device), out.to(device), w_next.to(device) if nxt else None,
                                  w2.to(device) if nxt else None, 1e-5, torch.float32)
        assert torch.allclose(xd.cpu(), new, rtol=1e-5, atol=1e-5)
        if nxt:
            u2 = sum(w_next[s] * new[:, s] for s in range(S)).double()
            assert torch.allclose(h2.cpu().double(), oracle.layer_norm(u2, w2, 1e-5), rtol=1e-4, atol=1e-4)
        else:
            assert h2 is None


@pytest.mark.parametrize("device", DEVICES)
def test_embed_streams_and_activations(device):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(0)
    table = torch.randn(11, 20, generator=g)
    ids = torch.tensor([3, 0, 10, 3], dtype=torch.int32)
    x = mixers.embed_streams(ids.to(device), table.to(device), 2.5, 3).cpu()
    assert x.shape == (4, 3, 20) and all(torch.equal(x[:, s], table[ids.long()] * 2.5) for s in range(3))
    z = torch.randn(3, 50, generator=g)
    assert torch.allclose(mixers.relu_sq(z.to(device)).cpu(), torch.relu(z) ** 2, rtol=1e-6, atol=1e-6)
    gu = torch.randn(3, 60, generator=g)
    want = torch.nn.functional.silu(gu[:, :30]) * gu[:, 30:]
    assert torch.allclose(mixers.silu_mul(gu.to(device)).cpu(), want, rtol=1e-5, atol=1e-6)


def _mlstm_case(H, D, Dv, cap, width=24, seed=0):
    cfg = make_config([mlstm_layer(heads=H, dim=D, vdim=Dv, gate_cap=cap)], width=width)
    T = oracle.random_tensors(cfg, seed)
    return cfg["layers"][0]["mixer"], {k[len("l0.mix."):]: v for k, v in T.items() if k.startswith("l0.mix.")}


def _mlstm_through_ops(m, P, hs, device, cuts, slot=1, slots=3):
    """The mixer assembled from the ops as the model does, rows fed in portions `cuts` (state carried in `slot`)."""
    from ai_agent_kubectl_amd.ops import mixers

    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    f32 = lambda t: t.float().to(device)   # noqa: E731
    w_proj = torch.cat([P["q"], P["k"], P["v"], P["g"]]).float().to(device)
    w_if, b_if = f32(torch.cat([P["i"], P["f"]])), f32(torch.cat([P["i.b"], P["f.b"]]))
    st = (torch.full((slots, H, Dv, D), 7.0, device=device), torch.full((slots, H, D), -3.0, device=device),
          torch.full((slots, H), 5.0, device=device))      # stale contents of a slot used before
    out, at = [], 0
    for c in cuts:
        h = hs[at:at + c].float().to(device)
        proj = h @ w_proj.t()
        gates = mixers.mlstm_gates(h, w_if, b_if, float(m.get("gate_cap") or 0.0))
        pos = torch.arange(at, at + c, dtype=torch.int32, device=device)
        o, den = mixers.mlstm_scan(proj, 0, H * D, 2 * H * D, gates, *st, torch.tensor([slot], dtype=torch.int32, device=device),
                                   torch.tensor([0, c], dtype=torch.int32, device=device), pos, H, D, Dv, D ** -0.5)
        y = mixers.headnorm_gate(o, proj, 2 * H * D + H * Dv, f32(P["norm"]), H, Dv, 1e-6, torch.float32, den)
        out.append((y @ f32(P["o"]).t()).cpu())
        at += c
    return torch.cat(out)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dv,cap", [(2, 8, 8, 15.0), (1, 5, 19, 0.0), (3, 33, 16, 2.0), (2, 64, 40, 15.0)])
def test_mlstm_recurrence(device, H, D, Dv, cap):
    m, P = _mlstm_case(H, D, Dv, cap)
    g = torch.Generator().manual_seed(5)
    hs = torch.randn(37, 24, generator=g).to(torch.bfloat16).double() * 1.5
    want = oracle.mlstm(hs, {"x." + k: v for k, v in P.items()}, "x.", m, 1e-6)
    for cuts in ([37], [1] * 37, [2, 16, 1, 17, 1]):     # whole, token by token, portions over the 16-row tiles
        got = _mlstm_through_ops(m, P, hs, device, cuts)
        assert torch.allclose(got.double(), want, rtol=2e-4, atol=2e-4), cuts


@pytest.mark.parametrize("device", DEVICES)
def test_mlstm_remembers_a_far_token_and_caps_its_gates(device):
    """The forget gates are pushed to stay open (large bias), one early token gets a large input gate: its value
    must still dominate the read-out 300 tokens later; without the cap the gates would differ by orders."""
    m, P = _mlstm_case(2, 8, 8, 6.0, seed=3)
    P["f.b"] = torch.full_like(P["f.b"], 30.0)        # capped to 6: f = logsigmoid(6), not logsigmoid(30)
    P["f"] = torch.zeros_like(P["f"])
    g = torch.Generator().manual_seed(6)
    hs = torch.randn(320, 24, generator=g).to(torch.bfloat16).double()
    want = oracle.mlstm(hs, {"x." + k: v for k, v in P.items()}, "x.", m, 1e-6)
    uncapped = oracle.mlstm(hs, {"x." + k: v for k, v in P.items()}, "x.", dict(m, gate_cap=None), 1e-6)
    assert not torch.allclose(uncapped[-1], want[-1], rtol=1e-2, atol=1e-3)
    got = _mlstm_through_ops(m, P, hs, device, [300] + [1] * 20)
    assert torch.allclose(got.double(), want, rtol=5e-4, atol=5e-4)


def _attention_case(device, m, n, seed=0, width=24, craft=None):
    """Latent attention of one layer assembled from the ops (cache pages shuffled) against the oracle."""
    from ai_agent_kubectl_amd.ops import mixers

    cfg = make_config([attention_layer(**m)], width=width)
    T = oracle.random_tensors(cfg, seed)
    if craft:
        craft(T)
    mm = cfg["layers"][0]["mixer"]
    g = torch.Generator().manual_seed(seed + 1)
    hs = torch.randn(n, width, generator=g).to(torch.bfloat16).double()
    want = oracle.latent_attention(hs, T, "l0.mix.", mm, 1e-6, oracle.latent_kv(hs, T, "l0.mix.", mm, 1e-6))
    H, D, Dr, Dv, Q, R = mm["heads"], mm["dim"], mm["rot_dim"], mm["vdim"], mm["q_rank"], mm["kv_rank"]
    f32 = lambda t: t.float().to(device)   # noqa: E731
    bs, nb = 16, (n + 15) // 16 + 3
    cache = torch.zeros((nb, bs, R + Dr), device=device)
    pages = torch.randperm(nb, generator=g)[: (n + 15) // 16].to(torch.int32)
    pos = torch.arange(n, dtype=torch.int32)
    slots = (pages[pos.long() // bs] * bs + pos % bs).to(torch.int32).to(device)
    pos = pos.to(device)
    rot = mm.get("rot")
    inv = f32(rot["base"] ** (-2.0 * torch.arange(rot["dims"] // 2, dtype=torch.float64) / rot["dims"])) if rot else f32(torch.zeros(0))
    rd = rot["dims"] if rot else 0
    h = f32(hs)
    proj = h @ f32(torch.cat([T["l0.mix.dq"], T["l0.mix.dkv"]])).t()
    cq = mixers.latent_prep(proj, Q, R, Dr, f32(T["l0.mix.dq.norm"]), f32(T["l0.mix.dkv.norm"]), inv, pos, slots, cache, rd, 1e-6)
    qn, qr = mixers.rope_split_q((cq @ f32(T["l0.mix.uq"]).t()).contiguous(), inv, pos, H, D, Dr, rd)
    q_lat = torch.bmm(qn, f32(T["l0.mix.uk"]).view(H, D, R))
    bt = pages.view(1, -1).to(device)
    outs = []
    for q_starts in (torch.tensor([0, n], dtype=torch.int32, device=device),):
        o_lat = mixers.window_attention(q_lat, qr, cache, bt, q_starts, pos, slots, f32(T["l0.mix.sink"]),
                                        (mm.get("mask") or {}).get("size", 0), mm["scale"])
        o = torch.bmm(o_lat, f32(T["l0.mix.uv"]).view(H, Dv, R).transpose(1, 2)).transpose(0, 1).reshape(n, H * Dv)
        outs.append((o @ f32(T["l0.mix.o"]).t()).cpu().double())
    return outs[0], want, T


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("m", [dict(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=12, kv_rank=16, window=8),
                               dict(heads=3, dim=5, rot_dim=6, vdim=9, q_rank=7, kv_rank=11, window=21),
                               dict(heads=5, dim=16, rot_dim=0, vdim=4, q_rank=8, kv_rank=24, window=0),
                               dict(heads=1, dim=4, rot_dim=8, vdim=4, q_rank=4, kv_rank=8, window=1),
                               dict(heads=70, dim=8, rot_dim=8, vdim=8, q_rank=16, kv_rank=120, window=40)])
def test_latent_attention_options(device, m):
    got, want, _ = _attention_case(device, m, 45)
    assert torch.allclose(got, want, rtol=3e-4, atol=3e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("gap,seen", [(11, True), (12, False)])
def test_window_edge_one_score_stands_out(device, gap, seen):
    """The sink is made negligible and the key `gap` positions back is the only one the last query likes: with
    window 12 it is seen at gap 11 and not at gap 12, and the output flips between its value and the others'."""
    m = dict(heads=2, dim=8, rot_dim=0, vdim=8, q_rank=12, kv_rank=16, window=12)

    def craft(T):
        T["l0.mix.sink"] = torch.full_like(T["l0.mix.sink"], -30.0)

    got, want, T = _attention_case(device, m, 40, seed=2, craft=craft)
    assert torch.allclose(got, want, rtol=3e-4, atol=3e-4)
    # the same rows with the window one larger / smaller must differ where it matters
    other = dict(m, window=12 + (0 if seen else 1))
    if not seen:
        got2, want2, _ = _attention_case(device, other, 40, seed=2, craft=craft)
        assert not torch.allclose(want2[gap:], want[gap:], rtol=1e-3, atol=1e-3)


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_the_weight(device):
    """A large learned sink leaves the keys almost no weight: the output shrinks towards 0; sink -inf-like: plain softmax."""
    m = dict(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=12, kv_rank=16, window=16)
    big, want_big, _ = _attention_case(device, m, 20, seed=4, craft=lambda T: T.__setitem__("l0.mix.sink", torch.tensor([30.0, 26.0])))
    none, want_none, _ = _attention_case(device, m, 20, seed=4, craft=lambda T: T.__setitem__("l0.mix.sink", torch.tensor([-40.0, -40.0])))
    assert torch.allclose(big, want_big, rtol=3e-4, atol=1e-5) and torch.allclose(none, want_none, rtol=3e-4, atol=3e-4)
    assert big.abs().max() < 1e-2 * none.abs().max()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (8, 3, 4, 2), (12, 4, 4, 3), (5, 1, 1, 1), (4, 4, 2, 2), (64, 6, 8, 3)])
def test_router_groups_and_correction(device, E, top, groups, keep):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(E)
    W = 40
    h = torch.randn(33, W, generator=g).to(torch.bfloat16).float()
    wr = (torch.randn(E, W, generator=g) * 0.5).to(torch.bfloat16).float()
    # corrections large enough to change the choice, some negative so that a masked 0 would beat them
    corr = (torch.randn(E, generator=g) * 0.3 - 0.3).to(torch.bfloat16).float()
    T = {"x.router": wr, "x.correction": corr}
    r = {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}}
    ids, w = mixers.moe_route(h.to(device), wr.to(device), corr.to(device), top, groups, keep)
    ids, w = ids.cpu(), w.cpu()
    changed = 0
    for t in range(h.shape[0]):
        wi, ww = oracle.route(h[t].double(), T, "x.", r)
        order = np.argsort(ids[t].numpy())
        worder = np.argsort(wi.numpy())
        assert sorted(ids[t].tolist()) == sorted(wi.tolist()), t
        assert np.allclose(w[t].numpy()[order], ww.numpy()[worder], rtol=1e-4, atol=1e-6)
        plain, _ = oracle.route(h[t].double(), {"x.router": wr}, "x.", {"experts": E, "top": top})
        changed += sorted(plain.tolist()) != sorted(wi.tolist())
    assert abs(float(w.sum(-1).mean()) - 1.0) < 1e-4
    if E > top:
        assert changed > 0      # groups and correction matter for these inputs


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("T_rows", [3, 70])      # the matrix-vector kernels / the sorted segments
def test_experts_weighted_sum(device, T_rows):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(T_rows)
    E, W, ff, top = 5, 24, 10, 2
    h = torch.randn(T_rows, W, generator=g)
    w_gu, w_dn = torch.randn(E, 2 * ff, W, generator=g) * 0.3, torch.randn(E, W, ff, generator=g) * 0.3
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T_rows)]).to(torch.int32)
    w = torch.rand(T_rows, top, generator=g)
    got = mixers.moe_experts(h.to(device), w_gu.to(device), w_dn.to(device), ids.to(device), w.to(device)).cpu()
    want = torch.zeros(T_rows, W, dtype=torch.float64)
    for t in range(T_rows):
        for k in range(top):
            e = int(ids[t, k])
            Tn = {"e.gate": w_gu[e, :ff], "e.up": w_gu[e, ff:], "e.down": w_dn[e]}
            want[t] += float(w[t, k]) * oracle.gated_expert(h[t].double(), Tn, "e.")
    assert torch.allclose(got.double(), want, rtol=2e-4, atol=2e-4)


# ---------------------------------------------------------------------------------------------------
# the model in the engine
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_whole_prompt(tmp_path, device, name):
    c, W, path = model_for(tmp_path, name)
    toks = tokens_for(c, 50)
    got = replay(session(path, device), toks, [50])
    assert rel_err(got, want_logits(c, W, toks)) < tol("float32")
    # the first tokens of a sequence, and a sequence of one token
    one = replay(session(path, device), toks[:1], [1])
    assert rel_err(one, want_logits(c, W, toks[:1])) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["base", "attention_first"])
def test_layer_trail(tmp_path, device, name):
    c, W, path = model_for(tmp_path, name, seed=2)
    toks = tokens_for(c, 23, seed=1)
    want = []
    oracle.forward(c, W, toks, lambda i, x: want.append(x.numpy()))
    sess = session(path, device)
    got = []
    sess.runner.model.layer_hook = lambda i, x: got.append(x[:len(toks)].cpu().numpy())
    replay(sess, toks, [len(toks)])
    assert len(got) == len(want) == len(c["layers"])
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.abs(a - b).max() < 2e-4 * max(1.0, np.abs(b).max()), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_decode_token_by_token(tmp_path, device, name):
    """A short prompt, then 70 tokens one at a time: over page borders (16) and past every window."""
    c, W, path = model_for(tmp_path, name, seed=1)
    toks = tokens_for(c, 75, seed=2)
    got = replay(session(path, device), toks, [5] + [1] * 70)
    assert rel_err(got, want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cuts", [("base", [2, 2, 3, 9, 2, 16, 1, 1, 15, 2]), ("attention_first", [5, 5, 2, 11, 17, 13]),
                                       ("plain_residual", [31, 2, 1, 2, 17]), ("one_stream", [16, 16, 16, 5])])
def test_portions(tmp_path, device, name, cuts):
    c, W, path = model_for(tmp_path, name, seed=3)
    toks = tokens_for(c, sum(cuts), seed=3)
    got = replay(session(path, device), toks, cuts)
    assert rel_err(got, want_logits(c, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_pages_and_slots_reused(tmp_path, device):
    """Six unequal requests through a pool of 112 tokens and 3 state slots: portions of some beside single tokens
    of others; a finished request's pages and slot go to the next one, whose state must start from zero."""
    c, W, path = model_for(tmp_path, "base", seed=4)
    sess = session(path, device, max_tokens=112, max_requests=3)
    lens = {"a": 40, "b": 9, "c": 33, "d": 21, "e": 30, "f": 17}
    toks = {k: tokens_for(c, n, seed=10 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: want_logits(c, W, v) for k, v in toks.items()}
    plan = [[("a", 7)], [("a", 2), ("b", 3)], [("a", 1), ("b", 1), ("c", 20)], [("a", 14), ("b", 1), ("c", 2)],
            [("b", 4), ("c", 1), ("a", 1)], [("c", 10), ("a", 15)], [("d", 21)], [("d", 0), ("e", 2)],
            [("e", 27), ("f", 16)], [("e", 1), ("f", 1)]]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, end = [], []
        for rid, n in step:
            if n == 0:
                continue
            part = toks[rid][at[rid]:at[rid] + n]
            entries.append({"id": rid, "tokens": part, "want": list(range(n))})
            at[rid] += n
            if at[rid] == lens[rid]:
                end.append(rid)
        out = sess.step(entries, end)
        o = 0
        for e in entries:
            got[e["id"]].append(out[o:o + len(e["tokens"])])
            o += len(e["tokens"])
    assert at == lens
    assert sess.sched.state_slots.num_free == 3 and sess.sched.bm.num_free == sess.sched.bm.num_blocks
    for k in lens:
        assert rel_err(np.concatenate(got[k]), want[k]) < tol("float32"), k


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_inside_a_long_window(tmp_path, device):
    """A window of 400 over 25 pages: the logits at the end depend on a token 390 back (inside) and not on one
    410 back (outside); both through a prompt portion and through decoded tokens."""
    c = make_config([attention_layer(heads=2, dim=8, rot_dim=4, vdim=8, q_rank=12, kv_rank=16, window=400, mlp=dense(16))],
                    width=16, vocab=64)
    W = oracle.random_tensors(c, 7)
    W["l0.mix.sink"] = torch.full_like(W["l0.mix.sink"], -20.0)
    path = write_checkpoint(tmp_path / "far", c, W)
    toks = tokens_for(c, 430, seed=5)
    want = want_logits(c, W, toks)
    got = replay(session(path, device, max_tokens=448), toks, [420] + [1] * 10)
    assert rel_err(got, want) < tol("float32")
    inside, outside = list(toks), list(toks)
    inside[429 - 390] = (toks[429 - 390] + 1) % 64
    outside[429 - 410] = (toks[429 - 410] + 1) % 64
    assert np.abs(want_logits(c, W, inside)[-1] - want[-1]).max() > 1e-6
    assert np.abs(want_logits(c, W, outside)[-1] - want[-1]).max() < 1e-9


@pytest.mark.parametrize("device", DEVICES)
def test_steps_that_want_nothing(tmp_path, device):
    c, W, path = model_for(tmp_path, "base", seed=5)
    toks = tokens_for(c, 30, seed=6)
    sess = session(path, device)
    assert sess.step([{"id": "r", "tokens": toks[:20], "want": []}], []).shape == (0, c["vocab"])
    got = sess.step([{"id": "r", "tokens": toks[20:], "want": [9]}], ["r"])
    assert rel_err(got, want_logits(c, W, toks)[-1:]) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_generate_greedy_through_scheduler(tmp_path, device):
    """Greedy generation through build_engine / generate_blocking: the scheduler chunks the prompts (12 tokens a
    step), admits at most as many requests as there are state slots and frees slots for the ones that wait."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    c, W, path = model_for(tmp_path, "base", seed=6)
    prompts = [tokens_for(c, n, seed=20 + n) for n in (5, 19, 1, 26, 8, 13)]
    eng = build_engine(EngineOptions(model=path, device=device, dtype="float32", max_batch=3, max_batched_tokens=12,
                                     max_model_len=64, kv_cache_tokens=256, graph_buckets=(1, 2, 3), use_graphs=False,
                                     safe_decode=False, ignore_eos=True))
    assert eng.scheduler.state_slots.num_slots == 3 and not eng.bm.prefix_caching
    seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True, safe_decode=False))
    for p, s in zip(prompts, seqs):
        toks = list(p)
        for _ in range(10):
            toks.append(int(np.argmax(want_logits(c, W, toks)[-1])))
        assert s.generated == toks[len(p):]
    assert eng.scheduler.state_slots.num_free == 3


def test_state_slots_follow_the_sequence():
    from ai_agent_kubectl_amd.engine.block_manager import BlockManager, NoFreeBlocks, StateSlots
    from ai_agent_kubectl_amd.engine.scheduler import Scheduler
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams, Sequence

    slots = StateSlots(2)
    sch = Scheduler(BlockManager(8, 16, enable_prefix_caching=False), max_batch=4, state_slots=slots)
    seqs = [Sequence(prompt_ids=[1, 2, 3], params=SamplingParams(max_new_tokens=0)) for _ in range(3)]
    sch.schedule_given([(seqs[0], 3), (seqs[1], 2)])
    assert {seqs[0].state_slot, seqs[1].state_slot} == {0, 1}
    with pytest.raises(NoFreeBlocks):
        sch.schedule_given([(seqs[2], 3)])
    sch.release(seqs[0])
    assert seqs[0].state_slot == -1 and slots.num_free == 1
    sch.schedule_given([(seqs[2], 3)])
    assert seqs[2].state_slot == 0
    sch.abort(seqs[1])
    assert slots.num_free == 1 and seqs[1].state_slot == -1


def test_config_reader(tmp_path):
    from ai_agent_kubectl_amd.models.config import KafilornConfig, get_config

    for name in VARIANTS:
        c, W, path = model_for(tmp_path, name)
        cfg = get_config(path)
        assert cfg.family == "kafilorn" and cfg.num_layers == len(c["layers"])
        assert KafilornConfig.from_dict(cfg.to_dict(), cfg.name) == cfg
    bad = variant("base")
    bad["layers"][2]["mixer"]["kv_from"] = 0          # an mLSTM layer has no latent to lend
    with pytest.raises(ValueError):
        KafilornConfig.from_dict(bad)
    bad = variant("base")
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        KafilornConfig.from_dict(bad)
    bad = variant("base")
    bad["layers"][1]["mlp"]["router"]["top"] = 5       # more than the kept groups hold
    with pytest.raises(ValueError):
        KafilornConfig.from_dict(bad)
    cfg = get_config("tiny-kafilorn")
    assert cfg.has_state and cfg.kv_bytes_per_token() == (48 + 8) * 2


def test_loader_checks_shapes(tmp_path):
    from ai_agent_kubectl_amd.models.config import get_config
    from ai_agent_kubectl_amd.models.weights import ParallelInfo, build_weights

    c, W, path = model_for(tmp_path, "base")
    W2 = dict(W)
    W2["l1.mix.uk"] = W["l1.mix.uk"][:-1]
    bad = write_checkpoint(tmp_path / "bad", c, W2)
    with pytest.raises((ValueError, RuntimeError)):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)
    del W2["l1.mix.uk"]
    bad = write_checkpoint(tmp_path / "bad2", c, W2)
    with pytest.raises(KeyError):
        build_weights(bad, get_config(bad), ParallelInfo(), dtype=torch.float32)


# ---------------------------------------------------------------------------------------------------
# GPU only: the bf16 engine and captured decode
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["base", "attention_first"])
def test_bf16_engine(tmp_path, name):
    c, W, path = model_for(tmp_path, name, seed=8)
    toks = tokens_for(c, 60, seed=8)
    want = want_logits(c, W, toks)
    for cuts in ([60], [17, 2, 25] + [1] * 16):
        got = replay(session(path, "cuda", dtype="bfloat16"), toks, cuts)
        assert bf16_close(got, want), (cuts, row_errs(got, want))


@pytest.mark.gpu
def test_wider_shapes_gpu(tmp_path):
    """Sizes nearer a real model's: 128-entry heads, a 256-wide latent, vector loads in the score loop, several
    value-column workgroups per mLSTM head, 32 experts."""
    c = make_config([mlstm_layer(heads=4, dim=128, vdim=96, mlp=dense(512)),
                     attention_layer(heads=8, dim=64, rot_dim=32, vdim=64, q_rank=192, kv_rank=256, window=48,
                                     mlp=moe(experts=32, top=4, ff=64, groups=(8, 3), shared=128)),
                     attention_layer(heads=8, dim=64, rot_dim=32, vdim=64, q_rank=192, kv_rank=256, window=200, kv_from=1)],
                    width=512, vocab=320, streams=4)
    W = oracle.random_tensors(c, 9)
    path = write_checkpoint(tmp_path / "wide", c, W)
    toks = tokens_for(c, 90, seed=9)
    want = want_logits(c, W, toks)
    got = replay(session(path, "cuda", dtype="float32"), toks, [70, 3] + [1] * 17)
    assert rel_err(got, want) < tol("float32")
    got = replay(session(path, "cuda", dtype="bfloat16"), toks, [70, 3] + [1] * 17)
    assert bf16_close(got, want), row_errs(got, want)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_decode_matches_eager(tmp_path, dtype):
    """Decode steps replayed from captured graphs (several replays with eager prefill steps between them) give
    the tokens of the eager engine."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    c, W, path = model_for(tmp_path, "base", seed=11)
    prompts = [tokens_for(c, n, seed=30 + n) for n in (7, 21, 3, 12, 9)]
    got = []
    for graphs in (False, True):
        eng = build_engine(EngineOptions(model=path, device="cuda", dtype=dtype, max_batch=4, max_model_len=96,
                                         kv_cache_tokens=512, graph_buckets=(1, 2, 4), use_graphs=graphs, safe_decode=False,
                                         ignore_eos=True))
        if graphs:
            eng.runner.capture_graphs(autotune=False)
            assert eng.runner.graphs
        seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True, safe_decode=False))
        got.append([s.generated for s in seqs])
        if graphs:
            assert eng.runner.stats["graph_replays"] > 0
    assert got[0] == got[1]


@pytest.mark.gpu
@pytest.mark.parametrize("H,R,Dr,window,decode", [(16, 128, 32, 40, False), (4, 64, 0, 0, False), (20, 256, 64, 100, False),
                                                  (3, 32, 32, 9, False), (6, 48, 16, 50, True),
                                                  (40, 512, 64, 333, False), (16, 128, 32, 40, True), (33, 160, 32, 17, True),
                                                  (8, 512, 64, 0, True)])
def test_window_attention_matrix_core_kernel(H, R, Dr, window, decode):
    """bf16 shapes the matrix-core kernel takes (heads below / at / above a 16-head tile and not multiples of it,
    latents of 64 .. 512, windows that are not multiples of the 16-key tiles, none, shuffled pages), as prompt
    portions of several sequences and as decode rows, against the torch reference on the same bf16 inputs."""
    from ai_agent_kubectl_amd.ops import mixers, reference as ref

    g = torch.Generator().manual_seed(H + R)
    lens = [70, 5, 130] if not decode else [1, 1, 1, 1]
    ctx = [200, 5, 300] if not decode else [97, 1, 260, 33]          # tokens in the cache after this step
    bs, mb = 16, 20
    nb = len(lens) * mb + 3
    cache = (torch.randn(nb, bs, R + Dr, generator=g) * 0.7).to(torch.bfloat16)
    bt = torch.randperm(nb, generator=g)[: len(lens) * mb].view(len(lens), mb).to(torch.int32)
    pos, slots, starts = [], [], [0]
    for i, (n, c) in enumerate(zip(lens, ctx)):
        for p in range(c - n, c):
            pos.append(p)
            slots.append(int(bt[i, p // bs]) * bs + p % bs)
        starts.append(starts[-1] + n)
    T = len(pos) + 3                                                  # three padding rows
    pos_t = torch.tensor(pos + [0] * 3, dtype=torch.int32)
    slots_t = torch.tensor(slots + [-1] * 3, dtype=torch.int32)
    q_lat = (torch.randn(H, T, R, generator=g) * 0.5).to(torch.bfloat16)
    q_rot = torch.randn(T, H, Dr, generator=g)
    sink = torch.randn(H, generator=g)
    q_starts = None if decode else torch.tensor(starts, dtype=torch.int32)
    if decode:
        T = len(lens)
        q_lat, q_rot, pos_t, slots_t = q_lat[:, :T].contiguous(), q_rot[:T].contiguous(), pos_t[:T], slots_t[:T]
    scale = (R + Dr) ** -0.5 * 2
    want = ref.window_attention(q_lat.float(), q_rot.to(torch.bfloat16).float(), cache.float(), bt, q_starts, pos_t, slots_t,
                                sink, window, scale)
    dev = lambda x: None if x is None else x.cuda()   # noqa: E731
    outs = {}
    for tile in (True, False):
        mixers.WINDOW_TILE = tile
        try:
            outs[tile] = mixers.window_attention(dev(q_lat), dev(q_rot), dev(cache), dev(bt), dev(q_starts), dev(pos_t),
                                                 dev(slots_t), dev(sink), window, scale).float().cpu()
        finally:
            mixers.WINDOW_TILE = True
    n_real = len(pos) if not decode else T
    for tile, got in outs.items():
        err = (got[:, :n_real] - want[:, :n_real]).abs().max() / want.abs().max()
        assert err < (1.5e-2 if tile else 1e-2), (tile, float(err))
        assert torch.all(got[:, n_real:] == 0)


@pytest.mark.gpu
@pytest.mark.parametrize("T_rows,top", [(3, 2), (40, 3), (300, 2)])
def test_experts_grouped_on_matrix_cores(T_rows, top):
    """bf16 decode-sized steps: rows grouped by expert (fewer / more than a 16-row tile per expert, an expert with
    no row at all) against the fp32 sum over the same bf16 weights."""
    from ai_agent_kubectl_amd.ops import mixers, reference as ref

    g = torch.Generator().manual_seed(T_rows)
    E, W, ff = 6, 64, 96
    h = torch.randn(T_rows, W, generator=g).to(torch.bfloat16)
    w_gu = (torch.randn(E, 2 * ff, W, generator=g) * 0.3).to(torch.bfloat16)
    w_dn = (torch.randn(E, W, ff, generator=g) * 0.3).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E - 1, generator=g)[:top] for _ in range(T_rows)]).to(torch.int32)   # expert 5 idle
    w = torch.rand(T_rows, top, generator=g)
    want = ref.moe_experts(h.float(), w_gu.float(), w_dn.float(), ids, w)
    got = mixers.moe_experts(h.cuda(), w_gu.cuda(), w_dn.cuda(), ids.cuda(), w.cuda()).cpu()
    assert (got - want).abs().max() < 2e-2 * want.abs().max()


@pytest.mark.gpu
@pytest.mark.parametrize("T_rows,W,H", [(5, 128, 2), (100, 256, 12), (33, 384, 40)])
def test_gates_on_matrix_cores(T_rows, W, H):
    from ai_agent_kubectl_amd.ops import mixers, reference as ref

    g = torch.Generator().manual_seed(W)
    h = torch.randn(T_rows, W, generator=g).to(torch.bfloat16)
    w = (torch.randn(2 * H, W, generator=g) * 0.2).to(torch.bfloat16)
    b = torch.randn(2 * H, generator=g)
    want = ref.mlstm_gates(h.float(), w.float(), b, 6.0)
    slow = mixers.mlstm_gates(h.cuda(), w.float().cuda(), b.cuda(), 6.0).cpu()
    fast = mixers.mlstm_gates(h.cuda(), w.float().cuda(), b.cuda(), 6.0, w.cuda()).cpu()
    assert torch.allclose(slow, want, rtol=1e-4, atol=1e-4) and torch.allclose(fast, want, rtol=1e-4, atol=1e-4)
