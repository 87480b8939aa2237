"""Vivepel in the engine against the plain oracle (tests/vivepel_oracle.py).

Every test makes its own small configuration and random (or crafted) weights, writes them as a
checkpoint folder (config.json + model.safetensors: the reader and the loader are under test too),
builds the engine on it and compares logits with the oracle's whole-sequence forward.  The same
bodies run on the CPU (the ops' torch references) and, marked `gpu`, on the HIP kernels in fp32 and
bf16.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import vivepel_oracle as oracle

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]


def write_checkpoint(path, config, W):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))
    return str(path)


def session(path, device, dtype="float32", max_tokens=256):
    from ai_agent_kubectl_amd.engine.trace import TraceSession

    return TraceSession(path, dtype=dtype, max_tokens=max_tokens, device=device)


def replay(sess, tokens, cuts, rid="r", end=True):
    """Feed `tokens` in portions of the sizes `cuts`; logits of every position [n, vocab]."""
    out, at = [], 0
    for i, c in enumerate(cuts):
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


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def tokens_for(config, n, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, config["vocab"], (n,), generator=g).tolist()


def want_logits(config, W, tokens):
    return oracle.forward(config, W, tokens)[0].numpy()


def variant(name):
    g = torch.Generator().manual_seed(1)
    if name == "base":                 # GQA 2, partial rotary, chunk 8 (half a page)
        return oracle.random_config(g, layers=2, width=64, vocab=272, groups=2)
    if name == "mha_full_rot":         # one key/value head per query head, rotary on the whole head, one norm group
        return oracle.random_config(g, layers=2, width=48, vocab=264, groups=1, heads=3, kv_heads=3, dim=8, vdim=8,
                                    rot={"base": 100.0, "dims": 8}, mask={"size": 5}, ff=40)
    if name == "mqa_no_ff":            # one key/value head in all, no feed-forward, chunk 24 (one and a half pages)
        return oracle.random_config(g, layers=3, width=60, vocab=256, groups=3, heads=4, kv_heads=1, dim=16, vdim=16,
                                    rot={"base": 5000.0, "dims": 4}, mask={"size": 24}, mlp=False)
    if name == "mixed_layers":         # every layer its own sizes and constants; one without feed-forward
        c = oracle.random_config(g, layers=3, width=64, vocab=288, groups=4)
        c["layers"][0]["mixer"].update(heads=2, kv_heads=1, dim=32, vdim=32, mask={"size": 16},
                                       rot={"base": 10.0, "dims": 32}, scale=0.11, softcap=3.0)
        c["layers"][1]["mlp"] = None
        c["layers"][2]["mixer"].update(heads=6, kv_heads=3, dim=8, vdim=8, mask={"size": 3}, rot={"base": 1e4, "dims": 2},
                                       scale=0.5, softcap=80.0)
        c["layers"][2]["mlp"]["ff"] = 100
        return c
    raise KeyError(name)


VARIANTS = ["base", "mha_full_rot", "mqa_no_ff", "mixed_layers"]


# ---------------------------------------------------------------------------------------------------
# each mechanism alone: ops.mixers (torch reference on CPU, HIP kernel on GPU) against the oracle
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("groups,width", [(1, 24), (2, 64), (3, 96), (8, 256)])
def test_group_rmsnorm(device, groups, width):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(groups)
    x = torch.randn(5, width, generator=g) * torch.linspace(0.1, 30, width)   # parts of very different size
    w = torch.rand(width, generator=g) + 0.5
    want = oracle.group_rms_norm(x, w, groups, 1e-5)
    got = mixers.group_rmsnorm(x.to(device), w.to(device), groups, 1e-5)
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5)
    if groups > 1:   # one norm over the whole row would be wrong here
        assert not torch.allclose(oracle.group_rms_norm(x, w, 1, 1e-5), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("with_next", [False, True])
def test_post_norm_residual(device, with_next):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(3)
    W, G = 96, 3
    x, y = torch.randn(4, W, generator=g), torch.randn(4, W, generator=g) * 7
    wp, ls, wn = (torch.rand(W, generator=g) + 0.5 for _ in range(3))
    want_x = x + ls * oracle.group_rms_norm(y, wp, G, 1e-6)
    r = x.clone().to(device)
    nxt = mixers.post_norm_residual(r, y.to(device), wp.to(device), ls.to(device), wn.to(device) if with_next else None,
                                    G, 1e-6)
    assert torch.allclose(r.cpu(), want_x, rtol=1e-5, atol=1e-5)
    if with_next:
        assert torch.allclose(nxt.cpu(), oracle.group_rms_norm(want_x, wn, G, 1e-6), rtol=1e-5, atol=1e-5)
    else:
        assert nxt is None


@pytest.mark.parametrize("device", DEVICES)
def test_polynorm(device):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(4)
    z = torch.randn(6, 200, generator=g) * 2
    coef = torch.tensor([0.7, -0.3, 0.2, 0.05])
    want = oracle.poly_norm(z, coef, 1e-6)
    got = mixers.polynorm(z.to(device), coef.to(device), 1e-6)
    assert torch.allclose(got.cpu(), want, rtol=1e-5, atol=1e-5)


def _paged(n_tokens, bs, extra=3, seed=0):
    """A block table over shuffled pages (so a wrong page shows) for one sequence of n_tokens."""
    nb = (n_tokens + bs - 1) // bs
    perm = torch.randperm(nb + extra, generator=torch.Generator().manual_seed(seed)).tolist()
    return perm[:nb], nb + extra


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,rot", [(4, 2, 16, 8), (3, 3, 8, 8), (2, 1, 96, 0), (5, 5, 40, 6)])
def test_headnorm_rope_append(device, H, G, D, rot):
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(D)
    T, bs, base = 21, 4, 300.0
    positions = list(range(7, 7 + T))
    table, nb = _paged(7 + T, bs)
    qk = torch.randn(T, (H + G) * D, generator=g)
    qw, kw = torch.rand(D, generator=g) + 0.5, torch.rand(D, generator=g) + 0.5
    inv = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32)
    slots = torch.tensor([table[p // bs] * bs + p % bs for p in positions], dtype=torch.int32)
    slots[3] = -1                                   # a padding row writes nothing
    kc = torch.zeros(nb, G, bs, D).to(device)
    vc = torch.zeros(nb, G, bs, D).to(device)
    q = mixers.headnorm_rope_append(qk.to(device), qw.to(device), kw.to(device), inv.to(device),
                                    torch.tensor(positions, dtype=torch.int32).to(device), slots.to(device), kc, vc,
                                    H, G, D, rot, 1e-6)
    x = qk.view(T, H + G, D)
    want_q = oracle.rotary(oracle.head_rms_norm(x[:, :H], qw, 1e-6), positions, rot, base) if rot else \
        oracle.head_rms_norm(x[:, :H], qw, 1e-6)
    want_k = oracle.rotary(oracle.head_rms_norm(x[:, H:], kw, 1e-6), positions, rot, base) if rot else \
        oracle.head_rms_norm(x[:, H:], kw, 1e-6)
    assert torch.allclose(q.cpu(), want_q, rtol=2e-5, atol=2e-5)
    for t, p in enumerate(positions):
        page, off = table[p // bs], p % bs
        if t == 3:
            assert float(kc[page, :, off].abs().max()) == 0.0 and float(vc[page, :, off].abs().max()) == 0.0
            continue
        assert torch.allclose(kc[page, :, off].cpu(), want_k[t], rtol=2e-5, atol=2e-5)
        assert torch.equal(vc[page, :, off].cpu(), x[t, H:])      # the value is the key as projected


def _attention_case(device, H, G, D, chunk, cap, sink, mix, positions_q, n_ctx, bs=4, seed=0, q=None, k=None, v=None,
                    dtype=torch.float32, max_q=0):
    """chunk_attention for queries at `positions_q` of one sequence holding n_ctx cached tokens, against
    a direct evaluation; returns (got, want)."""
    from ai_agent_kubectl_amd.ops import mixers

    g = torch.Generator().manual_seed(seed)
    table, nb = _paged(n_ctx, bs, seed=seed)
    k = torch.randn(n_ctx, G, D, generator=g) if k is None else k
    v = torch.randn(n_ctx, G, D, generator=g) if v is None else v
    q = torch.randn(len(positions_q), H, D, generator=g) if q is None else q
    q, k, v = (t.to(dtype).float() for t in (q, k, v))                            # what the kernel's dtype can hold
    kc, vc = torch.full((nb, G, bs, D), 1e3), torch.full((nb, G, bs, D), 1e3)    # unused slots: loud if read
    for j in range(n_ctx):
        kc[table[j // bs], :, j % bs] = k[j]
        vc[table[j // bs], :, j % bs] = v[j]
    bt = torch.tensor([table + [0] * 2], dtype=torch.int32)
    T = len(positions_q)
    pos = torch.tensor(positions_q, dtype=torch.int32)
    slots = torch.tensor([table[p // bs] * bs + p % bs for p in positions_q], dtype=torch.int32)
    scale = 0.3
    if T == 1:     # decode form: token t is block-table row t
        q_starts = None
    else:
        q_starts = torch.tensor([0, T], dtype=torch.int32)
    got = mixers.chunk_attention(q.to(device, dtype), kc.to(device, dtype), vc.to(device, dtype), bt.to(device),
                                 None if q_starts is None else q_starts.to(device), pos.to(device), slots.to(device),
                                 None if mix is None else mix.to(device), chunk, scale, cap, sink,
                                 max_q=max_q).float().cpu()
    rep = H // G
    want = torch.zeros(T, H, D)
    for t, p in enumerate(positions_q):
        vis = [j for j in range(n_ctx) if (oracle.chunk_visible(p, j, chunk) if chunk else j <= p)]
        wts = torch.zeros(H, len(vis))
        for h in range(H):
            s = torch.stack([(q[t, h] * k[j, h // rep]).sum() for j in vis]) * scale
            s = oracle.soft_cap(s, cap) if cap else s
            wts[h] = oracle.sink_softmax_row(s) if sink else torch.softmax(s, 0)
        if mix is not None:
            wts = mix @ wts
        for h in range(H):
            for c, j in enumerate(vis):
                want[t, h] += wts[h, c] * v[j, h // rep]
    return got.view(T, H, D), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,chunk,cap,sink,mixed", [(4, 2, 16, 8, 20.0, True, True), (3, 3, 8, 5, 0.0, True, False),
                                                        (2, 1, 32, 0, 5.0, False, True), (6, 2, 24, 70, 50.0, True, True),
                                                        (1, 1, 8, 1, 2.0, True, True)])
def test_chunk_attention_options(device, H, G, D, chunk, cap, sink, mixed):
    mix = (torch.eye(H) * 0.6 + torch.randn(H, H, generator=torch.Generator().manual_seed(9)) * 0.4) if mixed else None
    n = 90
    got, want = _attention_case(device, H, G, D, chunk, cap, sink, mix, list(range(60, n)), n)      # a prompt's portion
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-4)
    for p in (0, 1, chunk - 1 if chunk else 7, chunk if chunk else 8, n - 1):                        # decoded alone
        if p < 0:
            continue
        got, want = _attention_case(device, H, G, D, chunk, cap, sink, mix, [p], n)
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-4), p


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,chunk,cap,sink,mixed", [(6, 2, 96, 48, 45.0, True, True), (20, 4, 32, 24, 0.0, True, True),
                                                        (32, 8, 128, 40, 30.0, True, True), (3, 1, 64, 0, 5.0, False, False),
                                                        (5, 5, 32, 7, 9.0, True, True), (17, 17, 64, 1000, 20.0, True, True)])
def test_chunk_attention_tile_kernel(H, G, D, chunk, cap, sink, mixed):
    """bf16 prompt portions on the 16-row tile kernel (MFMA scores): portions that start and end inside
    chunks, pages and 16-row tiles, against the direct fp32 evaluation of the same bf16 inputs."""
    from ai_agent_kubectl_amd.ops import _hip

    assert _hip.require_mixers().ka_chunk_attention_tile_ok(H, G, D, D, 4) == 1
    mix = (torch.eye(H) * 0.6 + torch.randn(H, H, generator=torch.Generator().manual_seed(9)) * (0.4 / H ** 0.5)) if mixed else None
    for lo, n in ((0, 70), (37, 90), (63, 81), (5, 14)):
        got, want = _attention_case("cuda", H, G, D, chunk, cap, sink, mix, list(range(lo, n)), n, dtype=torch.bfloat16,
                                    max_q=n - lo, seed=lo)
        assert torch.allclose(got, want, rtol=2e-2, atol=2e-2), (lo, n, float((got - want).abs().max()))
        # the per-token kernel on the same inputs agrees too (max_q 0 keeps it off the tile kernel)
        got1, _ = _attention_case("cuda", H, G, D, chunk, cap, sink, mix, list(range(lo, n)), n, dtype=torch.bfloat16, seed=lo)
        assert torch.allclose(got, got1, rtol=2e-2, atol=2e-2)
    for p in (0, 1, 15, 16, 17, 47, 48, 89):         # one decoded row per workgroup on the same kernel
        got, want = _attention_case("cuda", H, G, D, chunk, cap, sink, mix, [p], 90, dtype=torch.bfloat16, seed=p)
        assert torch.allclose(got, want, rtol=2e-2, atol=2e-2), (p, float((got - want).abs().max()))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wide_model_attention(dtype):
    """64 heads of 128: more LDS and more accumulators than the small shapes use (the kernel with one
    workgroup per token; the tile kernel does not take this width)."""
    H, G, D = 64, 8, 128
    mix = torch.eye(H) * 0.6 + torch.randn(H, H, generator=torch.Generator().manual_seed(9)) * 0.05
    t = 1e-4 if dtype == torch.float32 else 2e-2
    got, want = _attention_case("cuda", H, G, D, 32, 30.0, True, mix, list(range(30, 36)), 36, dtype=dtype, max_q=6)
    assert torch.allclose(got, want, rtol=t, atol=t)
    got, want = _attention_case("cuda", H, G, D, 32, 30.0, True, mix, [35], 36, dtype=dtype)
    assert torch.allclose(got, want, rtol=t, atol=t)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("decode", [False, True])
def test_chunk_edges_one_score_stands_out(device, decode):
    """A key just inside the chunk must get (almost) all the weight when its score stands out; a key
    just outside, with a far larger score still, must get none.  Chunk 12 over pages of 4."""
    H, G, D, chunk, n = 2, 1, 16, 12, 40
    g = torch.Generator().manual_seed(5)
    k = torch.randn(n, G, D, generator=g) * 0.1
    v = torch.randn(n, G, D, generator=g)
    for p in (35, 36, 47 - 12, 24, 25):           # 36 and 24 start a chunk: they see only themselves
        q = torch.randn(1 if decode else 2, H, D, generator=g) * 0.1
        first = (p // chunk) * chunk
        k2 = k.clone()
        k2[first, 0] = 0
        k2[first, 0, 3] = 30.0                    # the first key of p's chunk: a large score
        if first > 0:
            k2[first - 1, 0] = 0
            k2[first - 1, 0, 3] = 90.0            # the key before it: larger still, but outside
        q[-1, :, 3] = 5.0
        positions = [p] if decode else [p - 1, p] if p - 1 >= first else [p, p]
        got, want = _attention_case(device, H, G, D, chunk, 0.0, True, None, positions, n, q=q, k=k2, v=v)
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-4)
        assert torch.allclose(got[-1, 0], v[first, 0], atol=1e-3)      # all weight on the first key of the chunk


@pytest.mark.parametrize("device", DEVICES)
def test_sink_takes_the_weight_when_scores_are_low(device):
    H, G, D, n = 2, 2, 8, 10
    k = torch.ones(n, G, D)
    v = torch.ones(n, G, D)
    q = -torch.ones(1, H, D) * 4          # every score is -0.3 * 32 = -9.6: the sink (score 0) dominates
    got, want = _attention_case(device, H, G, D, 16, 0.0, True, None, [n - 1], n, q=q, k=k, v=v)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-6)
    assert float(got.abs().max()) < 1e-2               # without the sink the output would be 1
    got, _ = _attention_case(device, H, G, D, 16, 0.0, False, None, [n - 1], n, q=q, k=k, v=v)
    assert torch.allclose(got, torch.ones_like(got), atol=1e-5)


# ---------------------------------------------------------------------------------------------------
# the engine (checkpoint reader, loader, scheduler's given steps, block manager, runner, model)
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_whole_prompt(tmp_path, device, name):
    config = variant(name)
    W = oracle.random_weights(config, seed=11)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device)
    toks = tokens_for(config, 45, seed=2)
    got = replay(sess, toks, [len(toks)])
    assert rel_err(got, want_logits(config, W, toks)) < tol("float32")
    one = replay(sess, toks[:1], [1])                 # a sequence of a single token
    assert rel_err(one, want_logits(config, W, toks[:1])) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["base", "mixed_layers"])
def test_layer_trail(tmp_path, device, name):
    """The residual stream after every layer, not only the logits."""
    config = variant(name)
    W = oracle.random_weights(config, seed=12)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device)
    toks = tokens_for(config, 19, seed=3)
    trail = []
    sess.runner.model.layer_hook = lambda li, x: trail.append(x.detach().float().cpu().clone())
    replay(sess, toks, [len(toks)])
    want = oracle.forward(config, W, toks)[1]
    assert len(trail) == len(config["layers"])
    for li, x in enumerate(trail):
        assert torch.allclose(x[:len(toks)], want[li], rtol=1e-4, atol=1e-4), li


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", VARIANTS)
def test_decode_token_by_token(tmp_path, device, name):
    """A short prompt, then 40 tokens one by one: over chunk edges and page borders, through the decode path."""
    config = variant(name)
    W = oracle.random_weights(config, seed=13)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device)
    toks = tokens_for(config, 47, seed=4)
    got = replay(sess, toks, [7] + [1] * 40)
    assert rel_err(got, want_logits(config, W, toks)) < tol("float32")
    got = replay(sess, toks[:20], [1] * 20)                      # decoded from the very first token on
    assert rel_err(got, want_logits(config, W, toks[:20])) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,cuts", [("base", [2, 2, 3, 9, 2, 16, 1, 1, 15, 2]), ("mha_full_rot", [5, 5, 2, 11, 17, 13]),
                                       ("mqa_no_ff", [23, 2, 24, 4]), ("mixed_layers", [3, 2, 2, 2, 32, 12])])
def test_portions(tmp_path, device, name, cuts):
    config = variant(name)
    W = oracle.random_weights(config, seed=14)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device)
    toks = tokens_for(config, sum(cuts), seed=5)
    got = replay(sess, toks, cuts)
    assert rel_err(got, want_logits(config, W, toks)) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_and_page_reuse(tmp_path, device):
    """Four unequal requests interleaved (portions beside single tokens, a request skipping steps), in
    a pool that only fits them because finished requests give their pages back; each position must
    match the request run alone (the oracle)."""
    config = variant("base")
    W = oracle.random_weights(config, seed=15)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device, max_tokens=112)
    reqs = {r: tokens_for(config, n, seed=20 + i) for i, (r, n) in enumerate([("a", 40), ("b", 9), ("c", 33), ("d", 26),
                                                                             ("e", 30), ("f", 17)])}
    plan = [[("a", 13), ("b", 2)], [("a", 1), ("b", 1), ("c", 20)], [("a", 1), ("c", 2), ("d", 26)],
            [("a", 25), ("b", 6), ("c", 1)], [("c", 10), ("e", 5)], [("e", 1), ("f", 17)], [("e", 24)]]
    at = {r: 0 for r in reqs}
    got = {r: [] for r in reqs}
    for step in plan:
        entries, end = [], []
        for r, n in step:
            entries.append({"id": r, "tokens": reqs[r][at[r]:at[r] + n], "want": list(range(n))})
            at[r] += n
            if at[r] == len(reqs[r]):
                end.append(r)
        out = sess.step(entries, end)
        o = 0
        for r, n in step:
            got[r].append(out[o:o + n])
            o += n
        assert o == out.shape[0]
    assert all(at[r] == len(reqs[r]) for r in reqs)
    assert sess.engine.bm.num_free == sess.engine.bm.num_blocks          # every page came back
    for r, toks in reqs.items():
        assert rel_err(np.concatenate(got[r]), want_logits(config, W, toks)) < tol("float32"), r


@pytest.mark.parametrize("device", DEVICES)
def test_far_key_in_long_chunk(tmp_path, device):
    """One layer whose weights make the query of the last token match one far key among a few hundred
    (chunk 512 over 16-token pages): the logits then depend on that key's value alone."""
    g = torch.Generator().manual_seed(6)
    config = oracle.random_config(g, layers=1, width=32, vocab=256, groups=1, heads=2, kv_heads=1, dim=16, vdim=16,
                                  rot={"base": 1e4, "dims": 0}, mask={"size": 512}, scale=1.0, softcap=40.0, mlp=False)
    W = oracle.random_weights(config, seed=16)
    W["l0.mix.talk"] = torch.eye(2).to(torch.bfloat16)
    W["l0.mix.q"] = (W["l0.mix.q"].float() * 6).to(torch.bfloat16)
    W["l0.mix.k"] = (W["l0.mix.k"].float() * 6).to(torch.bfloat16)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device, max_tokens=320)
    toks = tokens_for(config, 300, seed=7)
    want = want_logits(config, W, toks)
    got = replay(sess, toks, [290] + [1] * 10)
    assert rel_err(got[-12:], want[-12:]) < tol("float32")


@pytest.mark.parametrize("device", DEVICES)
def test_generate_greedy_through_scheduler(tmp_path, device):
    """Greedy generation through build_engine / generate_blocking: the scheduler chunks the prompts
    (a 12-token step budget), mixes them with decoding rows and frees pages; tokens match the oracle."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    config = variant("base")
    W = oracle.random_weights(config, seed=17)
    path = write_checkpoint(tmp_path / "m", config, W)
    eng = build_engine(EngineOptions(model=path, device=device, dtype="float32", max_batch=4, max_batched_tokens=12,
                                     max_model_len=96, kv_cache_tokens=160, graph_buckets=(1, 2, 4), safe_decode=False,
                                     ignore_eos=True, use_graphs=False))
    eng.scheduler.min_chunk = 2
    prompts = [tokens_for(config, n, seed=30 + n) for n in (5, 21, 9)]
    seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=10, ignore_eos=True, safe_decode=False))
    for p, s in zip(prompts, seqs):
        toks = list(p)
        for _ in range(10):
            toks.append(int(want_logits(config, W, toks)[-1].argmax()))
        assert s.generated == toks[len(p):]


@pytest.mark.parametrize("device", DEVICES)
def test_steps_that_want_nothing(tmp_path, device):
    """Portions whose logits nobody asks for (and a request that is ended right after its portion)
    still fill the cache; later positions match."""
    config = variant("base")
    W = oracle.random_weights(config, seed=22)
    sess = session(write_checkpoint(tmp_path / "m", config, W), device)
    toks = tokens_for(config, 30, seed=10)
    assert sess.step([{"id": "x", "tokens": toks[:11], "want": []}], []).shape == (0, config["vocab"])
    assert sess.step([{"id": "x", "tokens": toks[11:12], "want": []}, {"id": "y", "tokens": toks[:3], "want": []}],
                     ["y"]).shape[0] == 0
    got = sess.step([{"id": "x", "tokens": toks[12:], "want": [0, 17]}], ["x"])
    want = want_logits(config, W, toks)
    assert rel_err(got, want[[12, 29]]) < tol("float32")
    assert sess.engine.bm.num_free == sess.engine.bm.num_blocks


@pytest.mark.parametrize("device", DEVICES)
def test_layer_without_mask_rot_or_softcap_entries(tmp_path, device):
    """A mixer whose configuration leaves out the mask, the rotary entry and the soft cap: plain causal
    attention (still with the sink and the head mixing).  The oracle gets the equivalent explicit values."""
    config = variant("base")
    W = oracle.random_weights(config, seed=23)
    lean = json.loads(json.dumps(config))
    for L in lean["layers"][:1]:
        del L["mixer"]["mask"], L["mixer"]["rot"], L["mixer"]["softcap"]
    full = json.loads(json.dumps(config))
    full["layers"][0]["mixer"].update(mask={"size": 1 << 20}, rot={"base": 1.0, "dims": 0}, softcap=1e9)
    sess = session(write_checkpoint(tmp_path / "m", lean, W), device)
    toks = tokens_for(config, 40, seed=11)
    got = replay(sess, toks, [13, 2, 20] + [1] * 5)
    assert rel_err(got, want_logits(full, W, toks)) < tol("float32")


def test_settings_select_a_checkpoint_folder_and_dtype(tmp_path):
    from ai_agent_kubectl_amd.config import Settings
    from ai_agent_kubectl_amd.engine.builder import EngineOptions

    path = write_checkpoint(tmp_path / "m", variant("base"), oracle.random_weights(variant("base"), seed=1))
    opts = EngineOptions.from_settings(Settings(MODEL=path, DTYPE="float32"))
    assert opts.model == path and opts.dtype == "float32"


def test_config_reader_rejects_what_it_does_not_know(tmp_path):
    from ai_agent_kubectl_amd.models.config import get_config

    config = variant("base")
    config["layers"][0]["type"] = "recurrent"
    with open(tmp_path / "config.json", "w") as f:
        json.dump(config, f)
    with pytest.raises(ValueError):
        get_config(str(tmp_path))


# ---------------------------------------------------------------------------------------------------
# bf16 serving dtype and hipGraph decode (GPU only)
@pytest.mark.gpu
@pytest.mark.parametrize("name", ["base", "mixed_layers"])
def test_bf16_engine(tmp_path, name):
    config = variant(name)
    W = oracle.random_weights(config, seed=18)
    sess = session(write_checkpoint(tmp_path / "m", config, W), "cuda", dtype="bfloat16")
    toks = tokens_for(config, 50, seed=8)
    want = want_logits(config, W, toks)
    assert rel_err(replay(sess, toks, [len(toks)]), want) < tol("bfloat16")
    assert rel_err(replay(sess, toks, [3, 2, 20] + [1] * 25), want) < tol("bfloat16")


@pytest.mark.gpu
def test_bf16_engine_tile_kernel_shapes(tmp_path):
    """Head size 32 and portions of 8 rows and more: the engine's bf16 prompt steps run the tile kernel."""
    g = torch.Generator().manual_seed(2)
    config = oracle.random_config(g, layers=2, width=64, vocab=272, groups=2, heads=6, kv_heads=2, dim=32, vdim=32,
                                  rot={"base": 1000.0, "dims": 20}, mask={"size": 24}, scale=0.2, softcap=15.0)
    W = oracle.random_weights(config, seed=21)
    sess = session(write_checkpoint(tmp_path / "m", config, W), "cuda", dtype="bfloat16")
    toks = tokens_for(config, 75, seed=9)
    want = want_logits(config, W, toks)
    assert rel_err(replay(sess, toks, [len(toks)]), want) < tol("bfloat16")
    assert rel_err(replay(sess, toks, [9, 17, 30, 2, 16, 1]), want) < tol("bfloat16")
    # a mixed step: decode rows of two requests (the one-row form) beside a 40-row portion of a third (16-row tiles)
    other = tokens_for(config, 40, seed=12)
    sess.step([{"id": "a", "tokens": toks[:20], "want": []}, {"id": "b", "tokens": toks[:33], "want": []}], [])
    got = sess.step([{"id": "a", "tokens": toks[20:21], "want": [0]}, {"id": "c", "tokens": other, "want": list(range(40))},
                     {"id": "b", "tokens": toks[33:34], "want": [0]}], ["a", "b", "c"])
    assert rel_err(got[0:1], want[20:21]) < tol("bfloat16") and rel_err(got[41:42], want[33:34]) < tol("bfloat16")
    assert rel_err(got[1:41], want_logits(config, W, other)) < tol("bfloat16")


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["fp32_small_heads", "bf16_tile_kernel"])
def test_graph_decode_matches_eager(tmp_path, kind):
    """Captured decode graphs (replayed many times, with eager prompt steps between) give the eager
    tokens: the per-token attention kernel in fp32, and the tile kernel's one-row form in bf16 (head size
    32, more dynamic LDS than the default limit)."""
    from ai_agent_kubectl_amd.engine.builder import EngineOptions, build_engine
    from ai_agent_kubectl_amd.engine.sequence import SamplingParams

    if kind == "fp32_small_heads":
        config, dtype = variant("base"), "float32"
    else:
        g = torch.Generator().manual_seed(3)
        config = oracle.random_config(g, layers=2, width=64, vocab=272, groups=2, heads=20, kv_heads=4, dim=32, vdim=32,
                                      rot={"base": 1000.0, "dims": 16}, mask={"size": 24}, scale=0.2, softcap=15.0)
        dtype = "bfloat16"
    W = oracle.random_weights(config, seed=19)
    path = write_checkpoint(tmp_path / "m", config, W)
    prompts = [tokens_for(config, n, seed=40 + n) for n in (6, 17, 11)]
    outs = []
    for graphs in (False, True):
        eng = build_engine(EngineOptions(model=path, device="cuda", dtype=dtype, max_batch=4, max_model_len=96,
                                         kv_cache_tokens=256, graph_buckets=(1, 2, 4), safe_decode=False,
                                         ignore_eos=True, use_graphs=graphs))
        if graphs:
            eng.runner.capture_graphs()
        got = []
        for _ in range(2):      # a second wave reuses the freed pages and replays the same graphs
            seqs = eng.generate_blocking(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True, safe_decode=False))
            got.append([s.generated for s in seqs])
        if graphs:
            assert eng.runner.stats["graph_replays"] > 0
        assert got[0] == got[1]
        outs.append(got[0])
    assert outs[0] == outs[1]
