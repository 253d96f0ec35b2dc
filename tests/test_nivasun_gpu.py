"""Nivasun on the GPU against the plain implementation (``plain_nivasun``): every mechanism's kernels alone and as a
one-layer model, then the engine under schedules (whole, token by token, portions down to two tokens, unequal requests
in one batch, pages and state slots used again, long decoding) and greedy generation through ``LLM`` and the command
line.  Configurations and weights are the tests' own; where random weights would hide a fault (a key at a window's edge,
a sink, a temperature, the second of two maps), inputs are made so that it shows."""
import functools
import json
import math
import os
import tempfile
import types

import numpy as np
import pytest
import torch

import plain_nivasun as pn
from helpers import check

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TD = {"float32": torch.float32, "bfloat16": torch.bfloat16}
_keep = []


def T(a):
    return torch.as_tensor(np.asarray(a), dtype=torch.float64)


def close(got, want, dtype, what, scale=None):
    got, want = torch.as_tensor(got).double().cpu(), T(want)
    bound = (2e-5 if dtype == "float32" else 2e-2) * (float(want.abs().max()) if scale is None else scale)
    err = float((got - want.reshape(got.shape)).abs().max())
    assert err <= bound, f"{what}: {err:.3e} > {bound:.3e}"


def mostly(got, ref, dtype, what):
    """Every row against the plain logits: 32-bit to rounding; bfloat16 to a quarter of the spread everywhere and to a
    tenth at nine rows in ten (the tests' models are narrow, and a router may choose otherwise on a close call)."""
    ref = T(ref)
    if dtype == "float32":
        return check(got, ref, dtype, what)
    got = torch.as_tensor(got).double().reshape(ref.shape)
    err = (got - ref).abs().reshape(len(ref), -1).max(dim=1).values / float(ref.std())
    assert float(err.max()) <= 0.25, f"{what}: row {int(err.argmax())} is off by {float(err.max()):.3f} of the spread"
    over = int((err > 0.1).sum())
    assert over <= max(1, len(err) // 10), f"{what}: {over} of {len(err)} rows are off by more than a tenth of the spread"


def rnd(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(TD[dtype])


def step_of(ctx, qn, gpu, slots=None, page=8):
    """The index arrays of a step whose sequences have ``ctx`` tokens after it and bring ``qn`` of them."""
    cu = np.concatenate([[0], np.cumsum(qn)]).astype(np.int32)
    pos = np.concatenate([np.arange(c - n, c) for c, n in zip(ctx, qn)]).astype(np.int32)
    seq = np.concatenate([[i] * n for i, n in enumerate(qn)]).astype(np.int32)
    dec = [i for i, n in enumerate(qn) if n == 1]
    pre = [i for i, n in enumerate(qn) if n > 1]
    dev = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    return types.SimpleNamespace(
        positions=dev(pos), seq_of_token=dev(seq), cu_q=dev(cu), context_lens=dev(ctx), decode_seqs=dev(dec), prefill_seqs=dev(pre),
        state_slots=dev(slots if slots is not None else list(range(len(ctx)))), num_seqs=len(ctx), num_tokens=int(cu[-1]),
        n_decode=len(dec), n_prefill=len(pre), max_decode_context=max([ctx[i] for i in dec], default=0), max_q_len=max(qn),
        max_prefill_q=max([qn[i] for i in pre], default=0), min_prefill_prefix=min([ctx[i] - qn[i] for i in pre], default=0),
        page_size=page)


# ---- the embedding: a row by the token and the one before it; the token before a portion lives in a slot ------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,buckets,mp,mc", [(48, 37, 5, 11), (320, 1, 3, 2), (100, 64, 0, 1), (36, 1000, 70001, 99991), (64, 53, -7, 3)])
def test_pair_embedding_through_portions_and_slots(gpu, dtype, hidden, buckets, mp, mc):
    from prelude_amd.ops import kernels as K
    vocab = 75
    table, pair = rnd((vocab, hidden), 1, dtype), rnd((buckets + 1, hidden), 2, dtype)
    seqs = [torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(3 + n)).tolist() for n in (23, 1, 9)]
    want = [pn.embed(s, table.double().numpy(), 2.5, pair.double().numpy(), buckets, mp, mc) for s in seqs]
    prev = torch.full((5, 1), 12345, dtype=torch.int32, device=gpu)   # rubbish: a first token must not read it
    slots = [3, 0, 4]
    cuts = [[5, 1, 2, 15], [1], [2, 7]]            # the sequences' portions; step k brings the k-th of each that has one
    got = [[] for _ in seqs]
    fed = [0, 0, 0]
    for k in range(4):
        live = [i for i in range(3) if k < len(cuts[i])]
        qn = [cuts[i][k] for i in live]
        ids = sum((seqs[i][fed[i]: fed[i] + cuts[i][k]] for i in live), [])
        st = step_of([fed[i] + cuts[i][k] for i in live], qn, gpu, slots=[slots[i] for i in live])
        out = K.pair_embed(torch.tensor(ids, dtype=torch.int32, device=gpu), st, prev, table.to(gpu), pair.to(gpu), buckets, mp, mc, 2.5)
        assert out.dtype == torch.float32
        at = 0
        for i, n in zip(live, qn):
            got[i].append(out[at: at + n].cpu())
            at += n
            fed[i] += n
    for i in range(3):
        close(torch.cat(got[i]), want[i], "float32", f"sequence {i}")
    assert prev[slots[0], 0].item() == seqs[0][-1] and prev[1, 0].item() == 12345


# ---- the convolution over time in front of a mixer ------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,taps", [(48, 3), (320, 4), (36, 1), (257, 2), (64, 9)])
def test_time_convolution_carries_its_inputs_across_cuts(gpu, dtype, channels, taps):
    from prelude_amd.ops import kernels as K
    w = torch.randn((channels, taps), generator=torch.Generator().manual_seed(5)) * 0.5
    seqs = [rnd((n, channels), 6 + n, dtype) for n in (40, 3, 17)]
    want = [s.double().numpy() + pn.time_conv(s.double().numpy(), w.double().numpy()) for s in seqs]
    state = torch.full((4, max(taps - 1, 1), channels), 7.0, device=gpu) if taps > 1 else None
    if state is not None:
        state = state[:, : taps - 1].contiguous()
        state[[2, 0, 3]] = 0.0                     # what a request's start leaves; slot 1 keeps its rubbish
    slots = [2, 0, 3]
    cuts = [[1, 1, 2, 30, 1, 5], [3], [2, 2, 13]]
    got, fed = [[] for _ in seqs], [0, 0, 0]
    for k in range(6):
        live = [i for i in range(3) if k < len(cuts[i])]
        qn = [cuts[i][k] for i in live]
        h = torch.cat([seqs[i][fed[i]: fed[i] + cuts[i][k]] for i in live]).to(gpu)
        st = step_of([fed[i] + cuts[i][k] for i in live], qn, gpu, slots=[slots[i] for i in live])
        out = K.time_conv_add(h, w.t().contiguous().to(gpu), state, st)
        at = 0
        for i, n in zip(live, qn):
            got[i].append(out[at: at + n].cpu())
            at += n
            fed[i] += n
    for i in range(3):
        close(torch.cat(got[i]), want[i], dtype, f"sequence {i}")
    if state is not None:
        assert float(state[1].min()) == 7.0, "another request's slot is left alone"


@pytest.mark.parametrize("dtype", DTYPES)
def test_stream_adds_gate_and_cap(gpu, dtype):
    from prelude_amd.ops import kernels as K
    x = torch.randn((9, 100), generator=torch.Generator().manual_seed(1)) * 30
    a, b, row = rnd((9, 100), 2, dtype), rnd((9, 100), 3, dtype), torch.randn(100, generator=torch.Generator().manual_seed(4))
    s = x.clone().to(gpu)
    K.stream_add_branches_(s, a.to(gpu), b.to(gpu))
    close(s, x.double() + (a.double() + b.double()), "float32", "both branches")
    s = x.clone().to(gpu)
    K.stream_add_branches_(s, a.to(gpu))
    K.stream_add_row_(s, row.to(gpu))
    close(s, x.double() + a.double() + row.double(), "float32", "one branch and a row")
    wide = rnd((9, 260), 5, dtype)
    got = K.sigmoid_gate(a.to(gpu), wide.to(gpu)[:, 130: 230])
    close(got, a.double() * torch.sigmoid(wide[:, 130: 230].double()), dtype, "a gate out of a wider row")
    z = (torch.randn((5, 333), generator=torch.Generator().manual_seed(6)) * 20).to(gpu)
    close(K.cap_logits_(z.clone(), 7.5), 7.5 * torch.tanh(z.double().cpu() / 7.5), "float32", "capped logits")


# ---- rotation, cache write and attention over values that several key heads share; the two maps' difference -----------------
def _paged_read(kc, vc, table, n, page):
    """Keys [n, nk, hd] and values [n, nv, vd] of a sequence back out of its pages."""
    ks = torch.cat([kc[table[j]].transpose(0, 1) for j in range(-(-n // page))])[:n]
    vs = torch.cat([vc[table[j]].permute(2, 0, 1) for j in range(-(-n // page))])[:n]
    return ks, vs


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nk,nv,hd,vd,rot,pairs,page", [(8, 4, 2, 8, 24, 4, True, 8), (4, 2, 2, 32, 64, 16, True, 16),
                                                           (6, 2, 1, 16, 16, 16, False, 4), (2, 2, 1, 12, 40, 0, True, 8),
                                                           (3, 3, 3, 64, 64, 32, False, 16)])
def test_rotating_prepare_writes_queries_keys_and_values(gpu, dtype, nq, nk, nv, hd, vd, rot, pairs, page):
    from prelude_amd.ops import kernels as K
    n, base = 21, 777.0
    width = 5 + nq * hd + nk * hd + nv * vd
    p = rnd((n, width), 11, dtype)
    scale = 1 + 0.5 * torch.randn(nq, generator=torch.Generator().manual_seed(12))
    freq = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float64).float() if rot else None
    pos = list(range(100, 100 + n))
    layout = "pairs" if pairs else "halves"
    x = p.double().numpy()
    q_ref = x[:, 5: 5 + nq * hd].reshape(n, nq, hd)
    k_ref = x[:, 5 + nq * hd: 5 + (nq + nk) * hd].reshape(n, nk, hd)
    if rot:
        q_ref, k_ref = pn.rotate(q_ref, pos, rot, base, layout), pn.rotate(k_ref, pos, rot, base, layout)
    q_ref = q_ref * scale.double().numpy()[None, :, None]
    pages = -(-n // page) + 2
    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(13)).tolist()
    slots = torch.tensor([perm[i // page] * page + i % page for i in range(n)], dtype=torch.int32, device=gpu)
    kc = torch.zeros((pages, nk, page, hd), dtype=TD[dtype], device=gpu)
    vc = torch.zeros((pages, nv, vd, page), dtype=TD[dtype], device=gpu)
    q = K.qkv_rope_prepare(p.to(gpu), 5, 5 + nq * hd, 5 + (nq + nk) * hd, None if freq is None else freq.to(gpu),
                           torch.tensor(pos, dtype=torch.int32, device=gpu), slots, kc, vc, nq, nk, nv, hd, vd, rot, pairs,
                           q_scale=scale.to(gpu))
    close(q, q_ref, dtype, "queries", scale=float(np.abs(q_ref).max()))
    ks, vs = _paged_read(kc.cpu(), vc.cpu(), perm, n, page)
    close(ks, k_ref, dtype, "keys in their pages", scale=float(np.abs(k_ref).max()))
    assert torch.equal(vs.reshape(n, -1), p[:, 5 + (nq + nk) * hd:]), "values are copied as they are"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kvh,hd,vd,window,page", [(4, 2, 8, 24, 18, 8), (2, 2, 32, 64, 33, 16), (6, 1, 16, 16, 5, 4), (3, 3, 64, 128, 70, 16)])
def test_two_maps_over_shared_values_and_their_difference(gpu, dtype, heads, kvh, hd, vd, window, page):
    """2 * heads query heads over 2 * kvh key heads whose value head is the key head modulo kvh, map-major; one key
    just inside the window is made to take the second map's weight, so a second map that read the first map's keys, or
    a window one off, would show."""
    from prelude_amd.ops import kernels as K
    ctx, qn = [window + 30, 9, window], [window + 30, 1, 3]
    step = step_of(ctx, qn, gpu, page=page)
    lam, eps, out_scale, scale = 0.55, 1e-5, 0.7, 0.3
    qs, kcs, vcs, tables, wants = [], [], [], [], []
    g = torch.Generator().manual_seed(20)
    need = [-(-c // page) for c in ctx]
    total = sum(need) + 2
    perm = torch.randperm(total, generator=g).tolist()
    kc = torch.full((total, 2 * kvh, page, hd), 40.0, dtype=TD[dtype])
    vc = torch.full((total, kvh, vd, page), -40.0, dtype=TD[dtype])
    table = torch.full((3, max(need)), perm[-1], dtype=torch.int32)
    at = 0
    for s, (c, n) in enumerate(zip(ctx, qn)):
        k = (torch.randn((c, 2, kvh, hd), generator=g)).to(TD[dtype])     # [map][kv head]
        v = torch.randn((c, kvh, vd), generator=g).to(TD[dtype])
        q = (torch.randn((n, 2, heads, hd), generator=g)).to(TD[dtype])
        edge = c - window                      # the oldest key the last query sees
        if edge >= 0:
            k[edge, 1] = 3.0 * q[-1, 1, ::heads // kvh] / scale / hd ** 0.5
        for j in range(need[s]):
            pg = perm[at]
            at += 1
            table[s, j] = pg
            m = min(page, c - j * page)
            kc[pg, :, :m] = k[j * page: j * page + m].reshape(m, 2 * kvh, hd).transpose(0, 1)
            vc[pg, :, :, :m] = v[j * page: j * page + m].permute(1, 2, 0)
        qs.append(q.reshape(n, 2 * heads, hd))
        want = np.zeros((n, heads, vd))
        kk, vv, qq = k.double().numpy(), v.double().numpy(), q.double().numpy()
        for a in range(heads):
            gk = a // (heads // kvh)
            full_q = lambda mp: np.concatenate([np.zeros((c - n, hd)), qq[:, mp, a]])
            a1 = pn.windowed_softmax_sum(full_q(0), kk[:, 0, gk], vv[:, gk], scale, window)[c - n:]
            a2 = pn.windowed_softmax_sum(full_q(1), kk[:, 1, gk], vv[:, gk], scale, window)[c - n:]
            want[:, a] = pn.rms_unit(a1 - lam * a2, eps) * out_scale
        wants.append(want.reshape(n, heads * vd))
    group = types.SimpleNamespace(block_table=table.to(gpu))
    a = K.attention_masked(torch.cat(qs).to(gpu), kc.to(gpu), vc.to(gpu), group, step, window, 0, scale)
    got = K.diff_combine(a, heads, lam, eps, out_scale)
    close(got, np.concatenate(wants), dtype, "the maps' difference, normed", scale=1.0)


# ---- the router: the largest logits, the softmax over them alone ------------------------------------------------------------
@pytest.mark.parametrize("experts,top", [(6, 2), (16, 4), (3, 3), (70, 5), (2, 1)])
def test_router_by_logits_with_a_bias(gpu, experts, top):
    from prelude_amd.ops import kernels as K
    g = torch.Generator().manual_seed(30)
    z = torch.randn((41, experts + 1), generator=g) * 2
    bias = torch.randn(experts, generator=g) * 3          # large enough to change the choice
    choice, weights, gate = K.moe_route(z.to(gpu), experts, top, 1.0, None, gate_col=experts, bias=bias.to(gpu), by_logit=True)
    zb = (z[:, :experts] + bias).double()
    changed = 0
    for t in range(41):
        order = sorted(range(experts), key=lambda e: (-float(zb[t, e]), e))[:top]
        assert choice[t * top: (t + 1) * top].tolist() == order, f"token {t}"
        changed += order != sorted(range(experts), key=lambda e: (-float(z[t, e]), e))[:top]
        p = torch.softmax(zb[t, order], dim=0)
        assert float((weights[t * top: (t + 1) * top].double().cpu() - p).abs().max()) <= 1e-6
    assert changed or top == experts, "the bias decides somewhere"
    close(gate, torch.sigmoid(z[:, experts].double()), "float32", "the shared expert's gate")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,ff,experts,top,shared,tokens", [(48, 24, 6, 2, 40, 33), (64, 32, 3, 3, 0, 5), (36, 12, 2, 1, 12, 1), (128, 64, 8, 2, 64, 300)])
def test_routed_experts_part(gpu, dtype, hidden, ff, experts, top, shared, tokens):
    """The feed-forward as a part: with a wide margin between the router's logits in bfloat16 (its choice is not what
    this is about there)."""
    from prelude_amd.parts import build_part
    part = build_part("ffn", "routed_experts", dict(hidden_size=hidden, num_experts=experts, top=top, expert_size=ff, activation="silu",
                                                    router_bias=True, route="chosen_logits", correction=False, shared_size=shared))
    g = torch.Generator().manual_seed(31)
    w = {}
    for name, req in part.tensors().items():
        x = torch.randn(req.shape, generator=g) / math.sqrt(req.shape[-1])
        if name == "router.b":
            x = torch.randn(req.shape, generator=g)
        if name == "router" and dtype == "bfloat16":
            x = x * 30
        w[name] = x.to(torch.bfloat16)
    part.load({n: (t.to(TD[dtype]) if part.tensors()[n].kind == "matrix" else t.float()).to(gpu) for n, t in w.items()}, TD[dtype], gpu)
    x = rnd((tokens, hidden), 32, dtype)
    f = {"router": {"experts": experts, "top": top}, "shared": {"ff": shared} if shared else None}
    want = pn.routed_experts(x.double().numpy(), {n: t.double().numpy() for n, t in w.items()}, f)
    close(part.forward(x.to(gpu)), want, dtype, "experts", scale=float(np.abs(want).max()))


# ---- one-layer models ----------------------------------------------------------------------------------------------------
def write_model(cfg, w):
    from prelude_amd.weights import write_safetensors
    tmp = tempfile.TemporaryDirectory(prefix="prelude_amd_nivasun_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), {k: torch.as_tensor(v).to(torch.bfloat16) for k, v in w.items()})
    return tmp.name


def run_cut(path, dtype, toks, cuts, page=8, max_tokens=512):
    """The logits of every position with the sequence fed in portions of ``cuts`` (the rest one by one)."""
    from prelude_amd.trace import TraceRunner
    r = TraceRunner(path, dtype, max_tokens, page_size=page, state_slots=1)
    outs, i, k = [], 0, 0
    while i < len(toks):
        n = min(cuts[k], len(toks) - i) if k < len(cuts) else 1
        k += 1
        outs.append(r.step([{"id": "s", "tokens": toks[i:i + n], "want": list(range(n))}]))
        i += n
    return np.concatenate(outs)


def tokens(cfg, n, seed):
    return torch.randint(0, cfg["vocab"], (n,), generator=torch.Generator().manual_seed(seed)).tolist()


ONE_LAYER = [(pn.sink_layer, {}), (pn.sink_layer, dict(heads=3, kv_heads=3, dim=24, rot=0, window=7)),
             (pn.sink_layer, dict(heads=2, kv_heads=1, dim=64, rot=64, window=70, scale=0.125)),
             (pn.latent_layer, {}), (pn.latent_layer, dict(heads=2, dim=64, vdim=64, kv_rank=64, q_rank=16, window=33)),
             (pn.latent_layer, dict(heads=1, dim=8, vdim=40, kv_rank=12, q_rank=12, window=1)),
             (pn.diff_layer, {}), (pn.diff_layer, dict(heads=2, kv_heads=2, dim=32, vdim=64, rot=32, window=40)),
             (pn.diff_layer, dict(heads=3, kv_heads=1, dim=12, vdim=12, rot=0, window=3, diff=0.0))]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("make,over", ONE_LAYER)
def test_one_layer_whole_in_portions_and_token_by_token(gpu, dtype, make, over):
    cfg = pn.model([make(**over)], loop=(0, 1, 2))
    w = pn.random_weights(cfg, 50)
    toks = tokens(cfg, 130, 51)
    ref = pn.forward(cfg, w, toks)
    path = write_model(cfg, w)
    for cuts in ([130], [60], [7, 2, 13, 2, 1, 31, 2, 9, 16, 3, 8, 2, 30], []):
        mostly(run_cut(path, dtype, toks if cuts else toks[:60], cuts), ref if cuts else ref[:60], dtype, f"{make.__name__} {over} cut {cuts[:3]}")


@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("make,over,taps", [(pn.sink_layer, dict(window=24), 1), (pn.sink_layer, dict(window=16, heads=2, kv_heads=1, dim=64, rot=32), 3),
                                            (pn.latent_layer, dict(window=20), 1), (pn.latent_layer, dict(window=64), 2),
                                            (pn.diff_layer, dict(window=18), 1), (pn.diff_layer, dict(window=65, dim=32, vdim=64, rot=8), 4)])
def test_what_a_position_sees_ends_at_the_edge_of_its_window(gpu, make, over, taps, decoded):
    """A one-layer model: the key at j is made of the tokens j - taps .. j (the convolution's reach, and one more for the
    row the embedding takes by the token before).  So another token at c leaves the 32-bit logits at i as they are when
    c + taps < i - window + 1, and moves them as in the plain implementation when c + taps is the window's oldest key.
    For the last position of a prompt, and for a token decoded alone behind a prompt cut in the middle of a page."""
    window = over["window"]
    cfg = pn.model([make(**over)], taps=taps, loop=None)
    w = pn.random_weights(cfg, 60)
    path = write_model(cfg, w)
    n = 2 * window + 21
    toks = tokens(cfg, n, 61)
    i = n - 1
    cuts = [n - 19] if decoded else [n]

    def last(t):
        return run_cut(path, "float32", t, cuts)[-1]

    def other(c):
        t = list(toks)
        t[c] = (t[c] + 1 + c) % cfg["vocab"]
        return t
    base = last(toks)
    ref = pn.forward(cfg, w, toks)
    spread = float(ref.std())
    check(base, T(ref[-1]), "float32", "as it is")
    oldest = i - window + 1
    for c in (oldest - taps - 1, oldest - taps - 2):
        assert float(np.abs(last(other(c)) - base).max()) <= 1e-6 * spread, f"token {c} is outside what {i} sees"
    c = oldest - taps
    want = pn.forward(cfg, w, other(c))[-1]
    assert float(np.abs(want - ref[-1]).max()) > 1e-4 * spread, "the plain logits move"
    check(last(other(c)), T(want), "float32", f"token {c} is inside what {i} sees")


@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("make,over", [(pn.sink_layer, dict(window=40, heads=2, kv_heads=1, dim=64, rot=32, scale=0.125)),
                                       (pn.sink_layer, dict(window=80, heads=4, kv_heads=2, dim=64, rot=64, scale=0.125))])
def test_the_window_on_the_matrix_cores(gpu, make, over, decoded):
    """The same with heads of 64 under the bfloat16 engine, where this attention runs on the matrix cores: a changed token
    just outside leaves the logits bit for bit as they are; one just inside moves them as far as it moves the plain ones."""
    window, taps = over["window"], 1
    cfg = pn.model([make(**over)], taps=taps, loop=None)
    w = pn.random_weights(cfg, 62)
    path = write_model(cfg, w)
    n = 2 * window + 70
    toks = tokens(cfg, n, 63)
    i = n - 1
    cuts = [n - 19] if decoded else [n]

    def last(t):
        return run_cut(path, "bfloat16", t, cuts, page=16)[-1]

    def other(c):
        t = list(toks)
        t[c] = (t[c] + 1 + c) % cfg["vocab"]
        return t
    base = last(toks)
    ref = pn.forward(cfg, w, toks)
    oldest = i - window + 1
    for c in (oldest - taps - 1, oldest - taps - 2):
        assert np.array_equal(last(other(c)), base), f"token {c} is outside what {i} sees"
    c = oldest - taps
    moved = float(np.abs(pn.forward(cfg, w, other(c))[-1] - ref[-1]).max())
    got = float(np.abs(last(other(c)) - base).max())
    assert got > 0 and abs(got - moved) <= 0.5 * moved + 0.03 * float(ref.std()), f"token {c} is inside what {i} sees: {got} against {moved}"


@pytest.mark.parametrize("over,page", [(dict(heads=2, dim=64, vdim=64, kv_rank=64, q_rank=32, window=70), 16),
                                       (dict(heads=3, dim=32, vdim=64, kv_rank=40, q_rank=24, window=33), 8),
                                       (dict(heads=1, dim=128, vdim=128, kv_rank=96, q_rank=64, window=200), 16)])
def test_long_portions_attend_through_expanded_latents(gpu, over, page, monkeypatch):
    """Under the bfloat16 engine a long portion has every head's keys and values made from the latents it can see, in
    temporary pages, where short ones and single tokens attend to the latents themselves.  Both against the plain
    logits: whole, a long portion behind a prefix that ends inside a page (its window reaches back into the prefix), a long
    portion beside a sequence that decodes, and the same prompt with the expanded form switched off."""
    from prelude_amd.parts.latent_attention import LatentAttention
    from prelude_amd.trace import TraceRunner
    cfg = pn.model([pn.latent_layer(**over)], loop=(0, 1, 2), width=64)
    w = pn.random_weights(cfg, 80)
    toks, other = tokens(cfg, 700, 81), tokens(cfg, 60, 82)
    ref, ref_other = pn.forward(cfg, w, toks), pn.forward(cfg, w, other)
    path = write_model(cfg, w)
    used = []
    real = LatentAttention._expanded
    monkeypatch.setattr(LatentAttention, "_expanded", lambda self, *a: used.append(1) or real(self, *a))
    monkeypatch.setattr(LatentAttention, "EXPAND_FROM_TOKENS", 100)
    r = TraceRunner(path, "bfloat16", 1024, page_size=page, state_slots=2)
    mostly(r.step([{"id": "w", "tokens": toks, "want": list(range(700))}], ["w"]), ref, "bfloat16", "whole")
    assert len(used) == 2, "both runs of the layer expanded"
    outs = [r.step([{"id": "p", "tokens": toks[:53], "want": list(range(53))}])]
    assert len(used) == 2, "a short portion attends to the latents themselves"
    r.step([{"id": "o", "tokens": other[:40], "want": []}])
    outs.append(r.step([{"id": "p", "tokens": toks[53:400], "want": list(range(347))}]))
    both = r.step([{"id": "p", "tokens": toks[400:], "want": list(range(300))}, {"id": "o", "tokens": [other[40]], "want": [0]}])
    assert len(used) == 6
    mostly(np.concatenate(outs + [both[:300]]), ref, "bfloat16", "portions behind a prefix")
    mostly(both[300:], ref_other[40:41], "bfloat16", "a single token beside a long portion")
    monkeypatch.setattr(LatentAttention, "EXPAND_FROM_TOKENS", 1 << 30)
    r2 = TraceRunner(path, "bfloat16", 1024, page_size=page, state_slots=1)
    mostly(r2.step([{"id": "w", "tokens": toks, "want": list(range(700))}], ["w"]), ref, "bfloat16", "without the expanded form")
    assert len(used) == 6


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_sink_and_a_temperature_show(gpu, dtype):
    """Sinks far above the scores in every other head (those heads all but vanish, also at the first token, where a
    softmax without a sink gives the only key the weight 1), and temperatures far from 1."""
    cfg = pn.model([pn.sink_layer(heads=4, kv_heads=2, dim=16, window=24)], loop=None)
    w = pn.random_weights(cfg, 70)
    toks = tokens(cfg, 40, 71)
    ref0 = pn.forward(cfg, w, toks)
    w2 = dict(w)
    w2["l0.mix.sink"] = np.array([6.0, -3.0, 6.0, -3.0])
    w2["l0.mix.temp"] = np.array([1.0, 4.0, 0.25, 2.0])
    ref = pn.forward(cfg, w2, toks)
    assert float(np.abs(ref - ref0).max()) > 0.3 * float(ref.std()), "they matter"
    mostly(run_cut(write_model(cfg, w2), dtype, toks, [40]), ref, dtype, "whole")
    mostly(run_cut(write_model(cfg, w2), dtype, toks, []), ref, dtype, "token by token")


# ---- whole models ----------------------------------------------------------------------------------------------------------
CONFIGS = {"p": (pn.tiny_config_p, 11, 8), "q": (pn.tiny_config_q, 12, 16), "r": (pn.tiny_config_r, 13, 4)}
# The same three with every expert chosen ("pa", "qa", "ra"): what the bfloat16 engine is held to.  Between two experts
# whose logits nearly agree a router that sees bfloat16 inputs can choose the other one than the plain implementation in
# 64-bit, which is no fault and moves that row by more than the logits' spread (measured: a margin of 0.007 between
# logits of size 1.5, one row in a thousand choices), so no bound would tell it from a fault.  The choice itself is held
# in 32-bit by the configurations as they are, and in bfloat16 by the router's and the part's own tests.
for _n in "pqr":
    CONFIGS[_n + "a"] = CONFIGS[_n]


def named(name, dtype):
    return name + "a" if dtype == "bfloat16" else name


@functools.lru_cache(maxsize=None)
def folder(name):
    make, seed, _ = CONFIGS[name]
    cfg = make()
    if name.endswith("a"):
        for lc in cfg["layers"]:
            if lc.get("mlp"):
                lc["mlp"]["router"]["top"] = lc["mlp"]["router"]["experts"]
    w = pn.random_weights(cfg, seed)
    return write_model(cfg, w), cfg, w


@functools.lru_cache(maxsize=None)
def plain_logits(name, seed, length):
    _, cfg, w = folder(name)
    toks = tokens(cfg, length, 700 + seed)
    return toks, pn.forward(cfg, w, toks)


def runner(name, dtype, max_tokens, **kw):
    from prelude_amd.trace import TraceRunner
    return TraceRunner(folder(name)[0], dtype, max_tokens, page_size=CONFIGS[name][2], **kw)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_whole_prompt_every_position(gpu, name, dtype):
    name = named(name, dtype)
    toks, ref = plain_logits(name, 0, 200)
    r = runner(name, dtype, 256, state_slots=2)
    got = r.step([{"id": "x", "tokens": toks, "want": list(range(len(toks)))}], ["x"])
    mostly(got, ref, dtype, f"{name} whole")
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_every_run_of_the_stream(gpu, name):
    """The stream after every run of a layer (a looped layer counts each time), in 32-bit, against the plain one's."""
    toks, _ = plain_logits(name, 0, 200)
    _, cfg, w = folder(name)
    want = []
    pn.forward(cfg, w, toks[:60], streams=want)
    r = runner(name, "float32", 64, state_slots=1)
    seen = []
    for b in r.engine.model.blocks:
        def wrapped(*a, _f=b.forward, **k):
            h, res = _f(*a, **k)
            seen.append(res.clone())
            return h, res
        b.forward = wrapped
    r.step([{"id": "x", "tokens": toks[:60], "want": [59]}], ["x"])
    assert len(seen) == len(want) == len(pn.run_order(cfg))
    for i, (a, b) in enumerate(zip(seen, want)):
        close(a, b, "float32", f"after run {i}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_prefill_then_token_by_token(gpu, name, dtype):
    name = named(name, dtype)
    toks, ref = plain_logits(name, 1, 150)
    r = runner(name, dtype, 256, state_slots=1)
    n = 37                                  # a cut inside a page and inside every window
    outs = [r.step([{"id": 0, "tokens": toks[:n], "want": list(range(n))}])]
    for i in range(n, len(toks)):          # every window passes over decoded tokens; in bfloat16, replays of a captured step
        outs.append(r.step([{"id": 0, "tokens": [toks[i]], "want": [0]}]))
    mostly(np.concatenate(outs), ref, dtype, f"{name} decode")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_from_the_first_token_one_by_one(gpu, name, dtype):
    name = named(name, dtype)
    toks, ref = plain_logits(name, 2, 40)
    r = runner(name, dtype, 64, state_slots=1)
    outs = [r.step([{"id": 0, "tokens": [t], "want": [0]}]) for t in toks]
    mostly(np.concatenate(outs), ref, dtype, f"{name} one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_portions_of_changing_size(gpu, name, dtype):
    name = named(name, dtype)
    toks, ref = plain_logits(name, 3, 330)
    sizes = [7, 2, 13, 2, 1, 31, 2, 9, 16, 3, 8, 2, 64, 5, 129, 2]
    r = runner(name, dtype, 512, state_slots=1)
    outs, i, k = [], 0, 0
    while i < len(toks):
        n = min(sizes[k % len(sizes)], len(toks) - i)
        k += 1
        outs.append(r.step([{"id": "p", "tokens": toks[i:i + n], "want": list(range(n))}]))
        i += n
    mostly(np.concatenate(outs), ref, dtype, f"{name} portions")


def test_the_32_bit_logits_do_not_depend_on_the_cut(gpu):
    toks, _ = plain_logits("p", 4, 90)
    runs = []
    for cuts in ([90], [1] * 90, [5, 2, 40, 1, 22, 20]):
        r = runner("p", "float32", 128, state_slots=1)
        outs, i = [], 0
        for c in cuts:
            outs.append(r.step([{"id": "c", "tokens": toks[i:i + c], "want": list(range(c))}]))
            i += c
        runs.append(np.concatenate(outs))
    for other in runs[1:]:
        assert float(np.abs(other - runs[0]).max()) <= 5e-6 * float(np.abs(runs[0]).max())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["p", "q", "r"])
def test_unequal_requests_in_one_batch_with_pages_and_slots_used_again(gpu, name, dtype):
    name = named(name, dtype)
    """Six requests of unequal length through a pool that holds three of them and three state slots: portions of some
    beside single tokens of others; a request ends as soon as it is fed, and its pages and its slot (with the token and the
    convolutions' inputs it left there) go to the next."""
    lengths = [90, 17, 64, 33, 160, 5]
    seqs = [plain_logits(name, 10 + i, n) for i, n in enumerate(lengths)]
    r = runner(name, dtype, 3 * 192, state_slots=3)
    rng = np.random.default_rng(7)
    fed, waiting, live = [0] * len(seqs), list(range(len(seqs))), []
    got = [[] for _ in seqs]
    while waiting or live:
        while waiting and len(live) < 3:
            live.append(waiting.pop(0))
        entries, end = [], []
        for i in live:
            left = lengths[i] - fed[i]
            n = 1 if (fed[i] > 0 and rng.random() < 0.5) else int(min(left, rng.choice([2, 3, 16, 29, 40, 150])))
            entries.append({"id": f"r{i}", "tokens": seqs[i][0][fed[i]:fed[i] + n], "want": list(range(n))})
            fed[i] += n
            if fed[i] == lengths[i]:
                end.append(f"r{i}")
        out = r.step(entries, end)
        k = 0
        for e in entries:
            i = int(e["id"][1:])
            got[i].append(out[k:k + len(e["tokens"])])
            k += len(e["tokens"])
        live = [i for i in live if fed[i] < lengths[i]]
    for i, (toks, ref) in enumerate(seqs):
        mostly(np.concatenate(got[i]), ref, dtype, f"{name} request {i}")
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0
    assert r.engine.tables.free_state_slots() == 3


def test_a_batch_gives_what_each_request_gives_alone(gpu):
    """32-bit: a request's logits in a batch of unequal requests equal those it has alone, to rounding."""
    seqs = [plain_logits("p", 40 + i, n)[0] for i, n in enumerate([70, 9, 33])]
    alone = []
    for s in seqs:
        r = runner("p", "float32", 128, state_slots=1)
        alone.append(np.concatenate([r.step([{"id": 0, "tokens": s[:-4], "want": list(range(len(s) - 4))}])] +
                                    [r.step([{"id": 0, "tokens": [t], "want": [0]}]) for t in s[-4:]]))
    r = runner("p", "float32", 3 * 128, state_slots=3)
    first = r.step([{"id": i, "tokens": s[:-4], "want": list(range(len(s) - 4))} for i, s in enumerate(seqs)])
    tails = [r.step([{"id": i, "tokens": [s[len(s) - 4 + k]], "want": [0]} for i, s in enumerate(seqs)]) for k in range(4)]
    at = 0
    for i, s in enumerate(seqs):
        got = np.concatenate([first[at: at + len(s) - 4]] + [t[i:i + 1] for t in tails])
        at += len(s) - 4
        assert float(np.abs(got - alone[i]).max()) <= 5e-6 * float(np.abs(alone[i]).max()), f"request {i}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_token_far_back_moves_the_last_logits(gpu, dtype):
    """Every layer's window passes what it saw on to the next run, so a token some windows back still shows at the end; one
    beyond the reach of all runs together does not.  The engine follows the plain implementation in both."""
    name = named("p", dtype)                # windows of 24, 20, 18 (three times over) and 40, three taps
    toks, ref = plain_logits(name, 20, 260)
    _, cfg, w = folder(name)
    reach = 23 + 3 * (19 + 17) + 39 + 8 * 2 + 1
    near, far = 259 - 60, 259 - reach - 1
    for c, moves in ((near, True), (far, False)):
        other = list(toks)
        other[c] = (toks[c] + 1) % cfg["vocab"]
        ref2 = pn.forward(cfg, w, other)
        moved = float(np.abs(ref[-1] - ref2[-1]).max())
        assert (moved > 0.02 * float(ref.std())) == moves and (moves or moved == 0.0), f"the plain logits at the end, token {c}: {moved}"
        r = runner(name, dtype, 640, state_slots=2)
        assert r.step([{"id": "a", "tokens": toks[:129], "want": []}]) is None
        a = r.step([{"id": "a", "tokens": toks[129:], "want": [130]}], ["a"])
        b = r.step([{"id": "b", "tokens": other, "want": [259]}], ["b"])
        mostly(a, ref[-1:], dtype, "as it is")
        mostly(b, ref2[-1:], dtype, f"with token {c} changed")
        if not moves and dtype == "float32":
            assert float(np.abs(a - b).max()) <= 1e-6 * float(ref.std())


def test_a_request_longer_than_the_pool_holds(gpu):
    """Pages behind every window go back while the request lives: 600 tokens through a pool of 192, then long decoding."""
    name = "r"
    toks, ref = plain_logits(name, 21, 600)
    r = runner(name, "float32", 192, state_slots=1)
    outs, i = [], 0
    for n in [50, 3, 64] + [61] * 6 + [1] * 117:
        outs.append(r.step([{"id": "w", "tokens": toks[i:i + n], "want": list(range(n))}]))
        i += n
    assert i == 600
    check(np.concatenate(outs), T(ref), "float32", "a request longer than the pool")
    assert r.engine.tables.audit() == ""


def test_greedy_generation_through_the_scheduler(gpu):
    """``LLM.generate`` with temperature 0 gives the plain implementation's greedy tokens, for prompts of unequal length
    in one call (32-bit, so that no rounding decides between neighbours): the scheduler's portions, the token carried from
    one step to the next on the device, the slots."""
    from prelude_amd.llm import LLM
    name = "p"
    path, cfg, w = folder(name)
    llm = LLM(path, dtype="float32", page_size=8, max_cache_tokens=512)
    prompts = [plain_logits(name, 30, 9)[0], plain_logits(name, 31, 31)[0], plain_logits(name, 32, 2)[0]]
    res = llm.generate(prompts, max_tokens=12, temperature=0.0)
    for p, out in zip(prompts, res):
        seq = list(p)
        for _ in range(12):
            seq.append(int(pn.forward(cfg, w, seq)[-1].argmax()))
        assert out.token_ids == seq[len(p):], f"prompt of {len(p)}"


def test_greedy_generation_in_bfloat16_from_graphs(gpu):
    """The same through the serving path (bfloat16, steps replayed from captured graphs, the next step launched before
    the last one's tokens are read): each generated token is the plain implementation's choice given the tokens before
    it, wherever that choice is not a close call."""
    from prelude_amd.llm import LLM
    name = "qa"
    path, cfg, w = folder(name)
    llm = LLM(path, dtype="bfloat16", page_size=16, max_cache_tokens=1024)
    prompts = [plain_logits(name, 33, 20)[0], plain_logits(name, 34, 3)[0]]
    res = llm.generate(prompts, max_tokens=24, temperature=0.0)
    clear = 0
    for p, out in zip(prompts, res):
        assert len(out.token_ids) == 24
        seq = list(p) + out.token_ids
        ref = pn.forward(cfg, w, seq)
        for k in range(24):
            row = ref[len(p) - 1 + k]
            top2 = np.sort(row)[-2:]
            if top2[1] - top2[0] > 0.3 * float(row.std()):
                clear += 1
                assert out.token_ids[k] == int(row.argmax()), f"prompt of {len(p)}, token {k}"
    assert clear >= 10


def test_command_line_with_the_pools_sized_from_free_memory(gpu, capsys):
    from prelude_amd import cli
    name = "qa"
    path, cfg, w = folder(name)
    prompt = plain_logits(name, 40, 11)[0]
    assert cli.main(["--model", path, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "6", "--temperature", "0"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert rec["finish_reason"] == "length" and len(rec["token_ids"]) == 6
    ref = pn.forward(cfg, w, prompt)[-1]
    top2 = np.sort(ref)[-2:]
    if top2[1] - top2[0] > 0.25 * float(ref.std()):
        assert rec["token_ids"][0] == int(ref.argmax())
    assert cli.main(["--model", path, "--random-weights", "--prompt-len", "5", "--max-tokens", "3", "--max-cache-tokens", "256"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(rec["token_ids"]) == 3 and all(0 <= t < cfg["vocab"] for t in rec["token_ids"])


# ---- configurations drawn at random ------------------------------------------------------------------------------------
def draw_config(seed):
    """A Nivasun configuration drawn from a seed: any sizes the design allows, also ones no kernel is tuned for."""
    rng = np.random.default_rng(seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    window = lambda: int(pick([1, 2, 5, 16, 31, 32, 33, 64, 100]))

    def mlp():
        if rng.random() < 0.2:
            return None
        experts = int(pick([1, 2, 3, 5, 8, 16]))
        return pn._moe(int(pick([8, 16, 24, 40, 64])), experts, int(rng.integers(1, experts + 1)), int(pick([0, 8, 24, 48])))

    def rot(dim):
        return int(pick([0, 2, dim // 2, dim])) // 2 * 2

    layers = []
    for _ in range(int(rng.integers(2, 6))):
        kind = pick(["attention", "latent_attention", "attention_2"])
        kv, group = int(pick([1, 2, 3])), int(pick([1, 2, 4]))
        if kind == "attention":
            dim = int(pick([8, 16, 24, 32, 64, 128]))
            layers.append(pn.sink_layer(heads=kv * group, kv_heads=kv, dim=dim, window=window(), rot=rot(dim), base=float(pick([100.0, 1e4, 1e6])),
                                        scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim), mlp=mlp()))
        elif kind == "latent_attention":
            dim = int(pick([8, 16, 32, 64]))
            layers.append(pn.latent_layer(heads=kv * group, dim=dim, vdim=int(pick([8, 16, 24, 64])), kv_rank=int(pick([8, 12, 16, 40, 64, 96])),
                                          q_rank=int(pick([8, 12, 24, 64])), window=window(), scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim), mlp=mlp()))
        else:
            dim = int(pick([8, 16, 32, 64]))
            layers.append(pn.diff_layer(heads=kv * group, kv_heads=kv, dim=dim, vdim=2 * dim if rng.random() < 0.5 else int(pick([8, 16, 24, 40, 64])),
                                        window=window(), rot=rot(dim), base=float(pick([100.0, 1e4, 2e5])), scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim),
                                        diff=float(pick([0.0, 0.2, 0.5, 0.8])), mlp=mlp()))
    n = len(layers)
    loop = None
    if rng.random() < 0.8:
        start = int(rng.integers(0, n + 1))
        loop = (start, int(rng.integers(start, n + 1)), int(pick([1, 2, 3])))
    cfg = pn.model(layers, width=int(pick([32, 36, 48, 64, 72, 96, 128, 160])), vocab=int(rng.integers(40, 400)), loop=loop,
                   taps=int(pick([1, 2, 3, 4, 5])), buckets=int(pick([1, 7, 64, 521, 4099])), mul_prev=int(pick([0, 1, 31, 1009])),
                   mul_cur=int(pick([0, 1, 7, 997])), scale=float(pick([1.0, 4.0, 9.5])), cap=float(pick([0.0, 5.0, 15.0, 40.0])),
                   eps=float(pick([1e-6, 1e-5, 1e-4])))
    return cfg, int(pick([4, 8, 16, 32]))


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_CONFIGS", "12")))))   # widen for a hunt
def test_drawn_configuration(gpu, seed, monkeypatch):
    """Each drawn model whole, then in portions beside a request that decodes, through a pool and state slots that are
    used again: in 32-bit as drawn, in bfloat16 with every expert chosen (see ``CONFIGS``) and with portions of 64 tokens
    or more attending through expanded latents where the drawn head sizes allow it."""
    from prelude_amd.parts.latent_attention import LatentAttention
    from prelude_amd.trace import TraceRunner
    monkeypatch.setattr(LatentAttention, "EXPAND_FROM_TOKENS", 64)
    rng = np.random.default_rng(2000 + seed)
    for dtype in DTYPES:
        cfg, page = draw_config(seed)
        if dtype == "bfloat16":
            for lc in cfg["layers"]:
                if lc.get("mlp"):
                    lc["mlp"]["router"]["top"] = lc["mlp"]["router"]["experts"]
        toks = np.random.default_rng(2000 + seed).integers(0, cfg["vocab"], size=150).tolist()
        other = np.random.default_rng(3000 + seed).integers(0, cfg["vocab"], size=40).tolist()
        w = pn.random_weights(cfg, 300 + seed)
        ref, ref_other = pn.forward(cfg, w, toks), pn.forward(cfg, w, other)
        what = f"seed {seed} {dtype} page {page} {cfg}"
        r = TraceRunner(write_model(cfg, w), dtype, 256, page_size=page, state_slots=2)
        got = r.step([{"id": "w", "tokens": toks, "want": list(range(150))}], ["w"])
        mostly(got, ref, dtype, "whole: " + what)
        a, b, i, j = [], [], 0, 10
        r.step([{"id": "o", "tokens": other[:10], "want": []}])
        for n in (3, 70, 2, 17, 1, 1, 40, 16):
            entries = [{"id": "p", "tokens": toks[i:i + n], "want": list(range(n))}]
            if j < len(other):
                entries.append({"id": "o", "tokens": [other[j]], "want": [0]})
            out = r.step(entries)
            a.append(out[:n])
            if j < len(other):
                b.append(out[n:])
                j += 1
            i += n
        mostly(np.concatenate(a), ref[:i], dtype, "portions: " + what)
        mostly(np.concatenate(b), ref_other[10:j], dtype, "decoding beside them: " + what)
        assert r.engine.tables.audit() == ""
