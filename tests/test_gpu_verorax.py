"""Verorax through the engine against the plain float64 implementation (plain_verorax.py): every mechanism alone at
the level of its kernels or as a one-layer model, then whole models of made-up sizes in every way of cutting and
batching, 32-bit and bfloat16, and greedy generation through the engine's own entry point."""
import copy
import json
import random

import pytest
import torch

import plain_verorax as plain

pytestmark = pytest.mark.gpu
F = torch.float64


def latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, base=10000.0, scale=None):
    return dict(type="latent_attention", mixer=dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank,
                                                    q_rank=q_rank, scale=scale or (dim + rot_dim) ** -0.5,
                                                    rot=dict(base=base, dims=rot_dim)))


def differential(heads, kv_heads, dim, vdim, size, diff=0.25, scale=None):
    return dict(type="attention", mixer=dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale or dim ** -0.5,
                                             diff=diff, mask=dict(size=size)))


def parallel(lh, lg, ld, lv, size, dims, rh, rd, ls, rs, base=10000.0, scale=None):
    return dict(type="parallel", mixer=dict(
        left=dict(heads=lh, kv_heads=lg, dim=ld, vdim=lv, scale=scale or ld ** -0.5, mask=dict(size=size),
                  rot=dict(base=base, dims=dims)),
        right=dict(heads=rh, dim=rd), left_scale=ls, right_scale=rs))


def dense(layer, ff):
    return dict(layer, mlp=None if ff is None else dict(kind="dense", ff=ff))


def routed(layer, experts, identity, top, ff):
    return dict(layer, mlp=dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, identity=identity, top=top)))


def model(vocab, width, layers, eps=1e-6):
    return dict(architecture="Verorax", vocab=vocab, width=width, norm=dict(eps=eps), layers=layers)


L1 = latent(4, 16, 8, 24, 32, 24)                                   # values wider than the unrotated part
D1 = differential(4, 2, 8, 16, size=10)
P1 = parallel(4, 2, 16, 24, 7, 8, 2, 16, 0.7, 0.45)                 # half of a head rotated, values wider than keys
L2 = latent(3, 20, 12, 10, 24, 17, base=300.0)                      # sizes that are no multiples of 8, an odd head count
D2 = differential(3, 3, 20, 12, size=33, diff=0.0)                  # no group, nothing taken off but lambda
P2 = parallel(2, 2, 24, 24, 40, 24, 3, 40, 1.0, 1.0)                # the whole head rotated, scales of one
L3 = latent(8, 32, 16, 32, 64, 48)                                  # bfloat16: the latent attention on the matrix cores
D3 = differential(4, 1, 32, 64, size=5, diff=0.6)
P3 = parallel(4, 2, 64, 64, 9, 32, 2, 32, 0.25, 2.0)                # bfloat16: the left half on the matrix cores
P4 = parallel(6, 3, 8, 4, 3, 2, 1, 64, 0.8, 0.9)                    # one recurrent head, a window of three


def shared(layer, src):
    return dict(copy.deepcopy(layer), weights_of=src)


CONFIGS = {
    # every mixer, dense and routed feed-forwards, a layer without one, the last layer on layer 2's weights; pages of 4
    "V1": (model(96, 64, [dense(L1, 48), routed(D1, 6, 1, 2, 24), routed(P1, 6, 1, 2, 24), dense(L1, None),
                          shared(routed(P1, 6, 1, 2, 24), 2)]), 4, 11),
    # odd sizes; no identity expert and one choice; three identity experts of five outputs and three choices; another eps
    "V2": (model(131, 72, [routed(P2, 5, 0, 1, 40), routed(L2, 2, 3, 3, 56), dense(D2, 88)], eps=1e-3), 8, 12),
    # the model starts with layers that share weights; sizes the matrix-core kernels take; pages of 16
    "V3": (model(120, 128, [dense(P3, 96), shared(dense(P3, 96), 0), routed(L3, 8, 2, 2, 64), dense(D3, 64),
                            shared(dense(D3, 64), 3)]), 16, 13),
    # the second layer runs on the first's weights with another window and another diff, the fourth on the third's
    # with another scale and other shares of its halves
    "V4": (model(77, 40, [dense(D1, 24), dict(shared(dense(differential(4, 2, 8, 16, size=3, diff=0.5), 24), 0)),
                          dense(P4, 56), shared(dense(parallel(6, 3, 8, 4, 9, 2, 1, 64, 0.3, 1.1, scale=0.5), 56), 2)]), 4, 14),
}
# one mechanism a model (a parallel layer's other half scaled by zero)
ONE = {
    "latent": (model(64, 32, [dense(L1, None)]), 4, 21),
    "differential": (model(64, 32, [dense(D1, None)]), 4, 22),
    "left": (model(64, 32, [dense(parallel(4, 2, 16, 8, 6, 8, 2, 8, 1.0, 0.0), None)]), 4, 23),
    # bfloat16: heads of 64 rotated whole, which the 16-byte kernel before the cache takes (with the temperature)
    "left_whole": (model(64, 48, [dense(parallel(4, 2, 64, 64, 6, 64, 1, 8, 1.0, 0.0), None)]), 8, 27),
    "right": (model(64, 32, [dense(parallel(2, 1, 8, 8, 6, 4, 4, 24, 0.0, 1.0), None)]), 4, 24),
    "dense": (model(64, 32, [dense(parallel(2, 1, 8, 8, 6, 4, 2, 8, 0.0, 0.0), 72)]), 4, 25),
    "routed": (model(64, 32, [routed(parallel(2, 1, 8, 8, 6, 4, 2, 8, 0.0, 0.0), 7, 2, 3, 24)]), 4, 26),
}
# scores so sharp that one key too many or too few shows: windows of 6 and 4, pages of 4
SHARP = {
    "sharp": (model(80, 48, [dense(differential(2, 1, 16, 16, size=6, scale=1.5), 32),
                             dense(parallel(2, 1, 16, 16, 4, 8, 1, 8, 1.0, 0.0, scale=1.2), None),
                             dense(latent(2, 16, 8, 16, 24, 16, scale=1.0), None)]), 4, 31),
}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    from dinfer_amd.weights.safetensors_io import write_safetensors
    out = {}
    for name, (cfg, page, seed) in {**CONFIGS, **ONE, **SHARP}.items():
        d = tmp_path_factory.mktemp(f"verorax_{name}")
        w = plain.random_weights(cfg, seed, low=5 + seed % 4)
        (d / "config.json").write_text(json.dumps(cfg))
        write_safetensors(d / "model.safetensors", w, metadata={"format": "pt"})
        out[name] = (d, cfg, plain.as_float64(w), page)
    return out


def make_runner(models, name, dtype, max_tokens=512, num_blocks=160, max_seqs=4, max_len=512, graph=False):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    d, _, _, page = models[name]
    opt = EngineOptions(dtype=dtype, max_model_len=max_len, max_num_seqs=max_seqs, max_num_batched_tokens=max_tokens,
                        block_size=page, num_blocks=num_blocks, max_logits_rows=max_tokens,
                        decode_exempt_from_budget=False, hip_graph=graph)
    return ModelRunner.from_dir(d, opt)


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def has_router(cfg):
    return any((l.get("mlp") or {}).get("kind") == "moe" for l in cfg["layers"])


def check_logits(got, want, dtype, what, close_calls=False, sharp=False):
    got = got.double().cpu()
    scale = want.std(dim=-1, keepdim=True)
    err = ((got - want).abs() / scale).amax(dim=-1)
    rms = ((got - want).pow(2).mean(dim=-1, keepdim=True).sqrt() / scale).amax(dim=-1)
    if dtype == "float32":
        assert err.max().item() < 5e-4, f"{what}: 32-bit logits off by {err.max().item():.2e} row-sigmas"
        return
    # roundings to 8 bits through these narrow models add up to a few hundredths of a row's spread; a key too many or a
    # lost state is several times that. A router that reads rounded rows may choose another expert where two scores
    # nearly tie, which no arithmetic error is: in a model with routers one row in eight may be off by more.
    # sharp: scores of a spread of several units, whose rounding shows in the weights (a key too many still shows more)
    most, most_rms = (0.6, 0.25) if sharp else (0.3, 0.08)
    bad = (err >= most) | (rms >= most_rms)
    allowed = len(err) // 8 if close_calls else 0
    assert int(bad.sum()) <= allowed and err.max().item() < (2.5 if close_calls else most), \
        f"{what}: bf16 logits off by {err.max().item():.3f} (rms {rms.max().item():.4f}) row-sigmas, {int(bad.sum())} rows of {len(err)}"


def watch_routers(runner):
    """Every routed feed-forward of the runner's model notes what it chose, call by call (eager steps only)."""
    if not hasattr(runner, "routed_calls"):
        runner.routed_calls = []
        for ff in {id(b.ff): b.ff for b in runner.model.blocks if hasattr(b.ff, "idx")}.values():
            def noting(x, batch, _inner=ff.forward, _ff=ff, **kw):
                out = _inner(x, batch, **kw)
                runner.routed_calls.append(_ff.idx[:batch.num_tokens * _ff.top].cpu().view(-1, _ff.top).tolist())
                return out
            ff.forward = noting
    return runner.routed_calls


def replay(runner, steps, choices=None):
    """steps: [(entries, ends)], entries [(id, tokens, want)] -> {(id, position): logits row}.
    choices, a dict: receives {id: {(layer run, position): experts}}, what the engine's routers chose."""
    from dinfer_amd.engine.batch import Entry
    computed, rows = {}, {}
    calls = watch_routers(runner) if choices is not None else None
    routed_runs = [i for i, e in enumerate(runner.model.run) if hasattr(runner.model.blocks[e.layer].ff, "idx")]
    for entries, ends in steps:
        es = []
        for rid, toks, want in entries:
            start = computed.get(rid, 0)
            assert runner.reserve(rid, start, len(toks)), f"out of pages for {rid}"
            es.append(Entry(rid, toks, start, want))
        if es:
            if calls is not None:
                calls.clear()
            logits = runner.step(es).double().cpu()
            if calls is not None:
                assert len(calls) == len(routed_runs)
                for run, chosen in zip(routed_runs, calls):
                    at = 0
                    for e in es:
                        for k in range(len(e.tokens)):
                            choices.setdefault(e.req_id, {})[(run, e.start + k)] = chosen[at + k]
                        at += len(e.tokens)
            i = 0
            for e in es:
                for w in e.want:
                    rows[(e.req_id, e.start + w)] = logits[i]
                    i += 1
                computed[e.req_id] = e.start + len(e.tokens)
                runner.advance(e.req_id, computed[e.req_id])
        for rid in ends:
            runner.finish(rid)
            del computed[rid]
        runner.cache.check()
    return rows


def compare_rows(rows, cfg, w, toks, dtype, what, choices=None, sharp=False):
    """choices: what the engine's routers chose (replay). The plain model takes a choice over where the scores are so
    close that rounding the router's input may have turned it, and refuses any other; the rows are then compared as
    strictly as those of a model without routers. Without them (steps replayed from graphs, another process) a model
    with routers is allowed some rows that differ by more."""
    assert rows
    for rid in {k[0] for k in rows}:
        want = plain.forward(toks[rid.split("#")[0]], w, cfg, choices=(choices or {}).get(rid))
        pos = sorted(p for (r, p) in rows if r == rid)
        check_logits(torch.stack([rows[(rid, p)] for p in pos]), want[pos], dtype, f"{what} request {rid}",
                     has_router(cfg) and choices is None, sharp)


def run_and_compare(runner, steps, cfg, w, toks, dtype, what):
    choices = {} if dtype == "bfloat16" and has_router(cfg) else None
    rows = replay(runner, steps, choices)
    compare_rows(rows, cfg, w, toks, dtype, what, choices)
    return rows


def cut(ids, sizes):
    out, i, k = [], 0, 0
    while i < len(ids):
        out.append(ids[i:i + sizes[k % len(sizes)]])
        i += len(out[-1])
        k += 1
    return out


DTYPES = ["float32", "bfloat16"]
NAMES = list(CONFIGS)


# ---- one mechanism a model ------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(ONE))
def test_one_mechanism(models, name, dtype):
    """A model of one layer that is one mechanism (and the token shift before it): a whole prompt, the same in
    portions of two and three, and token by token."""
    _, cfg, w, _ = models[name]
    ids = tokens_for(cfg, 45, 3)
    r = make_runner(models, name, dtype)
    for what, parts in (("whole", [ids]), ("portions", cut(ids, [2, 3])), ("single tokens", [[t] for t in ids])):
        steps = [([("x", p, list(range(len(p))))], []) for p in parts]
        steps[-1] = (steps[-1][0], ["x"])
        run_and_compare(r, steps, cfg, w, {"x": ids}, dtype, f"{name} alone, {what}")


def test_token_shift_kernel_alone():
    """Portions of unequal length in one launch, among them a request's first tokens (zeros before them, whatever the
    slot holds), a portion of one row and a portion longer than a workgroup's rows; the kept rows afterwards."""
    from dinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(5)
    for dtype, width in ((torch.float32, 40), (torch.bfloat16, 264)):
        lens, starts, slots = [1, 19, 3, 8], [7, 0, 2, 0], [2, 0, 3, 1]
        T = sum(lens)
        x = torch.randn(T, width, generator=g).to(dtype)
        state = torch.randn(5, width, generator=g).to(dtype)
        mix = torch.rand(width, generator=g)
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
        seq = torch.tensor([s + n for s, n in zip(starts, lens)], dtype=torch.int32)
        out = torch.zeros(T, width, dtype=dtype, device="cuda")
        st = state.cuda()
        ops.token_shift(x.cuda(), out, st, mix.cuda(), cu_seqlens=cu.cuda(), seq_lens=seq.cuda(),
                        state_slots=torch.tensor(slots, dtype=torch.int32, device="cuda"), num_reqs=4, max_rows=max(lens))
        at = 0
        for n, s, slot in zip(lens, starts, slots):
            rows = x[at:at + n].double()
            first = state[slot].double() if s > 0 else torch.zeros(width, dtype=F)
            before = torch.cat([first[None], rows[:-1]])
            want = rows + (before - rows) * mix.double()
            tol = 1e-6 if dtype == torch.float32 else 2e-2
            assert (out[at:at + n].double().cpu() - want).abs().max().item() < tol
            assert torch.equal(st[slot].cpu(), x[at + n - 1])
            at += n
        assert torch.equal(st[4].cpu(), state[4])      # a slot of no request is left alone


def paged(rows, page, order):
    """rows [G, n, d] of one request -> (pages [blocks, G, page, d] with the request's pages in `order`, block table)."""
    G, n, d = rows.shape
    nb = -(-n // page)
    pages = torch.full((max(order) + 1, G, page, d), 7.0, dtype=rows.dtype)     # what no key owns holds junk, not zeros
    for i in range(nb):
        part = rows[:, i * page:(i + 1) * page]
        pages[order[i], :, :part.shape[1]] = part
    return pages, torch.tensor([order[:nb]], dtype=torch.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", [(4, 2, 16, 24, 4, 150, 20), (3, 3, 20, 12, 8, 200, 0), (2, 1, 32, 64, 16, 90, 7),
                                  (8, 1, 12, 8, 4, 70, 9)])
def test_differential_attention_kernel_alone(case, dtype):
    """The kernel on a made-up cache in shuffled pages. Each query's first map is a key of its request times a factor,
    so that one score stands out: far back, the oldest key the window still holds and the one before it, keys at a
    page's last and first place, and the query's own; the second map another key."""
    from dinfer_amd.kernels import ops
    H, G, D, V, page, n, window = case
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(n + D)
    k = torch.randn(G, n, 2 * D, generator=g).to(dt)
    v = torch.randn(G, n, V, generator=g).to(dt)
    p = n - 1
    wlo = max(0, p - window + 1) if window else 0
    targets = sorted({0, 1, wlo, max(wlo - 1, 0), p, p - 1, (p // page) * page, max((p // page) * page - 1, 0), n // 2})
    order = list(range(-(-n // page) + 3))
    random.Random(n).shuffle(order)
    kp, table = paged(k, page, order)
    vp, _ = paged(v, page, order)
    scale, lam, eps, post = 0.9 / D ** 0.5, 0.37, 1e-5, 0.7
    k_cache = ops.k_cache_pack(kp).cuda()
    v_cache = vp.permute(0, 1, 3, 2).contiguous().cuda()
    for target in targets:
        q = torch.randn(H, 2 * D, generator=g)
        for h in range(H):
            for m, tg in ((0, target), (1, (target * 7 + 3) % n)):
                key = k[h // (H // G), tg, m * D:(m + 1) * D].float()
                q[h, m * D:(m + 1) * D] += 6.0 * key / key.norm() * D ** 0.25
        q = q.to(dt)
        out = torch.zeros(1, H * V, dtype=dt, device="cuda")
        ops.attn_paged_diff(q.view(1, -1).cuda(), out, k_cache, v_cache, table.cuda(),
                            torch.tensor([0, 1], dtype=torch.int32, device="cuda"),
                            torch.tensor([n], dtype=torch.int32, device="cuda"), 1, 1, scale=scale, window=window, heads=H,
                            kv_heads=G, head_dim=D, v_dim=V, page_size=page, lam=lam, eps=eps, post=post)
        j = torch.arange(n)
        mask = ((j <= p) & (p - j < window)) if window else (j <= p)
        want = torch.zeros(H, V, dtype=F)
        for h in range(H):
            kv = h // (H // G)
            maps = [plain.softmax_rows(((k[kv, :, m * D:(m + 1) * D].double() @ q[h, m * D:(m + 1) * D].double()) * scale)[None],
                                       mask[None])[0] @ v[kv].double() for m in (0, 1)]
            want[h] = plain.rms_unit(maps[0] - lam * maps[1], eps) * post
        tol = 5e-5 if dtype == "float32" else 4e-2
        err = (out.double().cpu().view(H, V) - want).abs().max().item()
        assert err < tol * max(1.0, want.abs().max().item()), f"{case} target {target}: off by {err:.2e}"


@pytest.mark.parametrize("sizes", [(2, 8, 3), (1, 24, 5), (3, 40, 8), (2, 64, 6), (1, 136, 16), (1, 256, 4)])
def test_channel_delta_kernels_alone(sizes):
    """The recurrence's kernels on made-up projections: two requests in one launch, one from its first token and one
    that goes on from a state, in two steps; outputs and states against the rule written out token by token."""
    from dinfer_amd.kernels import ops
    H, D, low = sizes
    g = torch.Generator().manual_seed(D)
    hd = H * D
    lens = [(0, 21), (5, 3)]                 # (tokens before, tokens now)
    cols = 5 * hd + low
    a_b, w0 = torch.randn(hd, generator=g) * 0.8, torch.randn(hd, generator=g) * 0.8
    w2 = torch.randn(hd, low, generator=g) * (2.5 / low ** 0.5)
    state0 = torch.randn(3, H, D, D, generator=g) * 0.3            # [slot, head, value, key]
    rate, eps = 0.55, 1e-6
    for step in range(2):
        T = sum(n for _, n in lens)
        proj = torch.randn(T, cols, generator=g)
        work = torch.zeros(T, ops.channel_delta_work_columns(H, D), device="cuda")
        out = torch.zeros(T, hd, device="cuda")
        st = state0.clone().cuda()
        ops.channel_delta_prep(proj.cuda(), T, r_off=0, k_off=hd, v_off=2 * hd, a_off=4 * hd, low_off=5 * hd, a_bias=a_b.cuda(),
                               w2=w2.cuda(), w0=w0.cuda(), work=work, heads=H, dim=D, eps=eps, rate=rate)
        cu = torch.tensor([0, lens[0][1], T], dtype=torch.int32, device="cuda")
        seq = torch.tensor([a + b for a, b in lens], dtype=torch.int32, device="cuda")
        slots = torch.tensor([2, 0], dtype=torch.int32, device="cuda")
        ops.channel_delta_recurrence(work, st, out, state_slots=slots, cu_seqlens=cu, seq_lens=seq, num_reqs=2, heads=H, dim=D)
        at = 0
        for (before, n), slot in zip(lens, (2, 0)):
            x = proj[at:at + n].double()
            r, k, v = (x[:, i * hd:(i + 1) * hd].view(n, H, D) for i in range(3))
            a = torch.sigmoid(x[:, 4 * hd:5 * hd] + a_b.double()).view(n, H, D)
            w = torch.exp(-rate * torch.sigmoid(torch.tanh(x[:, 5 * hd:]) @ w2.double().T + w0.double())).view(n, H, D)
            u = k / torch.sqrt((k * k).sum(-1, keepdim=True) + eps)
            for h in range(H):
                S = state0[slot, h].double().T.clone() if before else torch.zeros(D, D, dtype=F)     # [key, value]
                for t in range(n):
                    S = w[t, h][:, None] * S - torch.outer(a[t, h] * u[t, h], u[t, h] @ S) + torch.outer(k[t, h], v[t, h])
                    want = S.T @ r[t, h]
                    got = out[at + t, h * D:(h + 1) * D].double().cpu()
                    assert (got - want).abs().max().item() < 2e-4 * max(1.0, want.abs().max().item()), f"{sizes} token {t}"
                assert (st[slot, h].double().cpu().T - S).abs().max().item() < 2e-4 * max(1.0, S.abs().max().item())
            at += n
        assert torch.equal(st[1].cpu(), state0[1])
        lens = [(21, 1), (8, 40)]            # the second step: one decoded token beside a longer portion


def test_routing_kernels_alone():
    """Softmax over all outputs, the choice moved by the correction, weights as the scores are; identity experts get
    no tiles and hand the input on in the sum."""
    from dinfer_amd.kernels import ops
    g = torch.Generator().manual_seed(9)
    for experts, identity, top, width, T in ((6, 1, 2, 32, 50), (5, 0, 1, 24, 9), (2, 3, 3, 40, 200), (70, 2, 4, 16, 33)):
        n_out = experts + identity
        x = torch.randn(T, width, generator=g)
        router = torch.randn(n_out, width, generator=g) * (3.0 / width ** 0.5)
        corr = torch.randn(n_out, generator=g) * 0.1
        idx = torch.zeros(T * top, dtype=torch.int32, device="cuda")
        share = torch.zeros(T * top, device="cuda")
        z = torch.zeros(T * (n_out + 1), device="cuda")
        ops.moe_route(x.cuda(), router.cuda(), None, idx, share, None, T, top, z, all_scores=True, correction=corr.cuda())
        s = torch.softmax(x.double() @ router.double().T, dim=-1)
        choice = s + corr.double()
        want = torch.topk(choice, top, dim=-1).indices
        got = idx.cpu().view(T, top).long()
        for t in range(T):
            srt = choice[t].sort(descending=True).values
            if (srt[:-1] - srt[1:])[:top].min().item() > 1e-5:          # a clear choice
                assert got[t].tolist() == want[t].tolist()
            assert (share.cpu().view(T, top)[t].double() - s[t][got[t]]).abs().max().item() < 1e-6
        y = torch.randn(T * top, width, generator=g)
        out = torch.zeros(T, width, device="cuda")
        ops.moe_combine(y.cuda(), share, top, None, None, out, T, idx=idx, real_experts=experts, x=x.cuda())
        sh = share.cpu().view(T, top).double()
        ref = torch.zeros(T, width, dtype=F)
        for t in range(T):
            for c in range(top):
                ref[t] += sh[t, c] * (x[t].double() if got[t, c] >= experts else y[t * top + c].double())
        assert (out.double().cpu() - ref).abs().max().item() < 1e-5
        offsets = torch.zeros(n_out + 1, dtype=torch.int32, device="cuda")
        perm = torch.zeros(T * top, dtype=torch.int32, device="cuda")
        tiles = torch.zeros((ops.moe_max_tiles(T * top, n_out, 16), 2), dtype=torch.int32, device="cuda")
        ops.moe_scatter(idx, T * top, n_out, offsets, perm, tiles, 16, real_experts=experts)
        named = tiles.cpu()[:, 0]
        assert named.max().item() < experts
        counts = torch.bincount(got.flatten(), minlength=n_out)
        for e in range(experts):
            assert int((named == e).sum()) == -(-int(counts[e]) // 16)


# ---- whole models ---------------------------------------------------------------------------------------------
def test_which_kernels_serve_which_model(models):
    """bfloat16 with sizes the matrix-core kernels take: those kernels for the latent attention and the left half of a
    parallel layer; 32-bit and other sizes: the plain kernels."""
    for name, dtype, mfma in (("V3", "bfloat16", True), ("V3", "float32", False), ("V2", "bfloat16", False)):
        r = make_runner(models, name, dtype)
        mixers = [b.mixer for b in r.model.blocks]
        lefts = [m for mx in mixers if hasattr(mx, "members") for _, m, _, _ in mx.members if hasattr(m, "mfma_ext")]
        latents = [m for m in mixers if hasattr(m, "attn_ws") and hasattr(m, "rank")]
        maps = [m for m in mixers if hasattr(m, "lam")]
        assert lefts and latents and maps
        assert all(m.mfma_ext == mfma for m in lefts) and all(bool(m.attn_ws.mfma) == mfma for m in latents)
        assert all(m.mfma == mfma for m in maps)       # (V2: values that are not twice a map's keys wide)


def test_layers_that_share_weights_have_caches_of_their_own(models):
    r = make_runner(models, "V1", "float32")
    assert [e.layer for e in r.model.run] == [0, 1, 2, 3, 2] and [e.cache for e in r.model.run] == [0, 1, 2, 3, 4]
    a, b = r.cache_views[2], r.cache_views[4]
    assert a.owner and b.owner and set(a.tensors) == set(b.tensors) == {"mixer.left.k", "mixer.left.v", "mixer.right.state",
                                                                         "mixer.right.conv", "shift.state"}
    assert all(a.tensors[k].data_ptr() != b.tensors[k].data_ptr() for k in a.tensors if a.tensors[k].numel())
    assert not r.cache.prefix_caching       # rows kept between steps cannot be found again in pages


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompts(models, name, dtype):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    for n, seed in ((1, 1), (2, 2), (19, 3), (150, 4)):
        ids = tokens_for(cfg, n, seed)
        run_and_compare(r, [([("x", ids, list(range(n)))], ["x"])], cfg, w, {"x": ids}, dtype, f"{name} whole prompt of {n}")


@pytest.mark.parametrize("name", NAMES)
def test_residual_stream_after_every_layer_run(models, name):
    from dinfer_amd.engine.batch import Entry
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, "float32")
    ids = tokens_for(cfg, 37, 9)
    want = []
    plain.forward(ids, w, cfg, want)
    seen = []
    for block in r.model.blocks:
        inner = block.forward

        def spy(hidden, pending, batch, cache, _inner=inner, **kw):
            out = _inner(hidden, pending, batch, cache, **kw)
            seen.append(hidden[:batch.num_tokens].double().cpu())
            return out
        block.forward = spy
    assert r.reserve("x", 0, len(ids))
    r.step([Entry("x", ids, 0, [0])])
    assert len(seen) == len(want) == len(cfg["layers"])
    for i, (g, x) in enumerate(zip(seen, want)):
        assert (g - x).abs().max().item() < 2e-4 * max(1.0, x.abs().max().item()), f"{name}: the stream after layer run {i} differs"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_prompt_then_long_decoding(models, name, dtype):
    """Decoding far beyond every window of the model, across many pages, from eager steps."""
    _, cfg, w, page = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 3 * page + 120, 5)
    first = 3 * page - 1                      # the first decoded token opens a new page
    steps = [([("x", ids[:first], [first - 1])], [])]
    steps += [([("x", [ids[p]], [0])], []) for p in range(first, len(ids))]
    run_and_compare(r, steps, cfg, w, {"x": ids}, dtype, f"{name} decode after prompt")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_token_by_token_from_the_first(models, name, dtype):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 60, 6)
    run_and_compare(r, [([("x", [t], [0])], []) for t in ids], cfg, w, {"x": ids}, dtype, f"{name} one token a step")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("sizes", [[2], [7, 16, 2, 5, 3, 33, 2, 8, 1], [64, 3, 31]])
def test_portions(models, name, dtype, sizes):
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype)
    ids = tokens_for(cfg, 131 if sizes != [2] else 48, 7)
    steps = [([("x", part, list(range(len(part))))], []) for part in cut(ids, sizes)]
    run_and_compare(r, steps, cfg, w, {"x": ids}, dtype, f"{name} portions of {sizes}")


def test_cuts_leave_the_same_logits_in_32bit(models):
    """32-bit: whole, in portions and token by token, a position's logits are equal to the last bits."""
    _, cfg, w, _ = models["V1"]
    ids = tokens_for(cfg, 70, 8)
    got = []
    for parts in ([ids], cut(ids, [5, 2, 11, 1]), [[t] for t in ids]):
        r = make_runner(models, "V1", "float32")
        rows = replay(r, [([("x", p, list(range(len(p))))], []) for p in parts])
        got.append(torch.stack([rows[("x", p)] for p in range(len(ids))]))
    for other in got[1:]:
        assert (other - got[0]).abs().max().item() < 2e-5 * got[0].abs().max().item()


def mixed_schedule(cfg, seed):
    """Four live requests at most: portions of some beside single tokens of others, requests that pause, finish and are
    followed by new ones in their pages and slots."""
    rng = random.Random(seed)
    lens = {"a": 90, "b": 33, "c": 57, "d": 21, "e": 70, "f": 12, "a#2": 90}
    toks = {k: tokens_for(cfg, n, sum(map(ord, k.split("#")[0]))) for k, n in lens.items()}
    order, live, at, steps = list(lens), [], {}, []
    while order or live:
        while order and len(live) < 4:
            k = order.pop(0)
            live.append(k)
            at[k] = 0
        entries, ends = [], []
        for k in list(live):
            if rng.random() < 0.2 and len(live) > 1:
                continue                                      # left out of this step
            left = lens[k] - at[k]
            n = min(left, rng.choice([1, 1, 1, 2, 3, 9, 17, 40]))
            entries.append((k, toks[k][at[k]:at[k] + n], sorted(rng.sample(range(n), min(n, 3)))))
            at[k] += n
            if at[k] == lens[k]:
                ends.append(k)
                live.remove(k)
        if entries:
            steps.append((entries, ends))
    return toks, steps


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_reused_pages_and_slots(models, name, dtype):
    _, cfg, w, page = models[name]
    toks, steps = mixed_schedule(cfg, 3)
    # fewer pages than all requests together need, and as many state slots as live requests: both are used again
    r = make_runner(models, name, dtype, num_blocks=(90 + 70 + 57 + 33) // page + 12, max_len=96)
    rows = run_and_compare(r, steps, cfg, w, toks, dtype, f"{name} mixed")
    if dtype == "float32":      # each request alone gives the same rows
        alone = replay(make_runner(models, name, dtype), [([("b", toks["b"], list(range(33)))], ["b"])])
        for (rid, p), row in rows.items():
            if rid == "b":
                assert (row - alone[("b", p)]).abs().max().item() < 1e-4 * row.abs().max().item()


# ---- edges that random weights would hide -------------------------------------------------------------------------
def with_windows(cfg, change):
    out = copy.deepcopy(cfg)
    for l in out["layers"]:
        m = l["mixer"].get("left", l["mixer"])
        if "mask" in m:
            m["mask"]["size"] += change
    return out


@pytest.mark.parametrize("dtype", DTYPES)
def test_keys_just_inside_and_outside_the_windows(models, dtype):
    """Scores so sharp that the oldest key a window holds often carries most of a row's weight. The engine agrees
    with the windows as configured, in a prompt and in decoding, and the same model with windows one key longer or
    shorter gives rows that differ by far more than the tolerance, so a window one key off could not pass."""
    _, cfg, w, page = models["sharp"]
    ids = tokens_for(cfg, 90, 2)
    want = plain.forward(ids, w, cfg)
    spread = want.std(dim=-1, keepdim=True)
    for change in (-1, 1):
        off = ((plain.forward(ids, w, with_windows(cfg, change)) - want).abs() / spread).amax(dim=-1)
        assert (off[8:] > 0.6).float().mean().item() > 0.5, "the made-up weights do not show a window that is one key off"
    r = make_runner(models, "sharp", dtype)
    whole = replay(r, [([("x", ids, list(range(len(ids))))], ["x"])])
    compare_rows(whole, cfg, w, {"x": ids}, dtype, "sharp whole", sharp=True)
    steps = [([("y", ids[:11], list(range(11)))], [])] + [([("y", [t], [0])], []) for t in ids[11:]]
    compare_rows(replay(r, steps), cfg, w, {"y": ids}, dtype, "sharp decoded", sharp=True)
    compare_rows(replay(r, [([("z", p, list(range(len(p))))], []) for p in cut(ids, [3, 2, 7])]), cfg, w, {"z": ids}, dtype,
                 "sharp in portions across the windows' edges", sharp=True)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_key_far_back_among_hundreds(models, dtype):
    """The latent attention sees everything: with sharp scores rows far into a long request take most of their weight
    from single keys hundreds of tokens back; without the keys more than 64 back the rows would be others."""
    _, cfg, w, page = models["sharp"]
    ids = tokens_for(cfg, 420, 4)
    want = plain.forward(ids, w, cfg)

    def near_only(T, size=None, _v=plain.visible):
        return _v(T, 64 if size is None else size)
    plain.visible, keep = near_only, plain.visible
    try:
        cut_off = plain.forward(ids, w, cfg)
    finally:
        plain.visible = keep
    off = ((cut_off - want).abs() / want.std(dim=-1, keepdim=True)).amax(dim=-1)
    assert (off[100:] > 0.6).float().mean().item() > 0.5, "the made-up weights do not show far keys"
    r = make_runner(models, "sharp", dtype)
    probe = [70, 200, 419]
    steps = [([("x", ids[:300], [70, 200])], [])] + [([("x", [t], [0])], []) for t in ids[300:]]
    rows = replay(r, steps)
    compare_rows(rows, cfg, w, {"x": ids}, dtype, "far keys", sharp=True)
    assert all(("x", p) in rows for p in probe)


def test_pages_behind_the_window_are_given_back(models):
    _, cfg, w, page = models["V4"]      # windows 10, 3, 3 and 9, pages of 4: every layer's pages are given back
    r = make_runner(models, "V4", "float32", num_blocks=110, max_len=400)
    ids = tokens_for(cfg, 300, 4)
    rows = replay(r, [([("x", p, [len(p) - 1])], []) for p in cut(ids, [9, 1, 1, 30, 2])])
    compare_rows(rows, cfg, w, {"x": ids}, "float32", "V4 long request")
    assert len(r.group_specs) == 4
    for g, spec in enumerate(r.group_specs):
        held = [i for i, pg in enumerate(r.cache.block_table("x", g)) if pg >= 0]
        assert held == list(range((len(ids) - spec.window + 1) // page, (len(ids) - 1) // page + 1))


# ---- graphs and the engine's own entry point ----------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["V1", "V3"])
def test_decode_steps_from_graphs(models, name, dtype):
    """Steps of single rows replay captured graphs (batch sizes 1 to 3, requests of unequal length, padded rows that
    use the spare state slot)."""
    _, cfg, w, _ = models[name]
    r = make_runner(models, name, dtype, graph=True)
    assert r._graphs_allowed
    ids = {k: tokens_for(cfg, n, s) for k, n, s in (("a", 60, 1), ("b", 45, 2), ("c", 70, 3))}
    steps = [([("a", ids["a"][:30], [29]), ("b", ids["b"][:5], [4])], []), ([("c", ids["c"][:41], [40])], [])]
    at = {"a": 30, "b": 5, "c": 41}
    while any(at[k] < len(ids[k]) for k in ids):
        es, ends = [], []
        for k in ids:
            if at[k] < len(ids[k]):
                es.append((k, [ids[k][at[k]]], [0]))
                at[k] += 1
                if at[k] == len(ids[k]):
                    ends.append(k)
        steps.append((es, ends))
    rows = replay(r, steps)
    assert r._graphs, "no decode graph was captured"
    # the same steps run eagerly agree with the plain model, and the replayed graphs with them
    eager = run_and_compare(make_runner(models, name, dtype), steps, cfg, w, ids, dtype, f"{name} eager decode")
    tol = 1e-5 if dtype == "float32" else 2e-2
    for key, row in rows.items():
        assert (row - eager[key]).abs().max().item() < tol * max(1.0, eager[key].abs().max().item()), f"{name} graph decode {key}"


@pytest.mark.parametrize("name", ["V1", "V2"])
def test_greedy_generation_through_the_engine(models, name):
    from dinfer_amd import Engine, SamplingParams
    d, cfg, w, page = models[name]
    eng = Engine(str(d), dtype="float32", max_model_len=256, max_num_seqs=3, block_size=page, num_blocks=120,
                 max_num_batched_tokens=64)
    prompts = [tokens_for(cfg, n, s) for n, s in ((5, 1), (70, 2), (23, 3), (1, 4))]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
    for prompt, out in zip(prompts, outs):
        ids = list(prompt)
        for tok in out:
            logits = plain.forward(ids, w, cfg)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3 * logits.std().item():     # a clear choice
                assert tok == int(logits.argmax()), f"{name}: greedy token differs after {len(ids)} tokens"
            ids.append(tok)


def test_bfloat16_generation_is_the_same_from_graphs(models):
    from dinfer_amd import Engine, SamplingParams
    d, cfg, _, page = models["V1"]
    prompts = [tokens_for(cfg, 40, s) for s in range(1, 9)] + [tokens_for(cfg, n, 20 + n) for n in (9, 3)]
    outs = []
    for graphs in (True, False):
        eng = Engine(str(d), dtype="bfloat16", max_model_len=128, max_num_seqs=2, block_size=page, num_blocks=96,
                     max_num_batched_tokens=16, hip_graph=graphs, gemm_tuning="heuristic")
        outs.append(eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0)))
        if graphs:
            assert eng.runner._graphs
    assert outs[0] == outs[1]


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay_program(models, tmp_path, dtype):
    """bin/trace_run on a made-up model: two requests in mixed steps; its files hold the rows the plain model gives."""
    import subprocess
    import sys
    from pathlib import Path
    import numpy as np
    d, cfg, w, _ = models["V1" if dtype == "float32" else "V4"]     # (bfloat16: a model without routers, see compare_rows)
    ids = {"a": tokens_for(cfg, 40, 1), "b": tokens_for(cfg, 9, 2)}
    lines = [dict(step=0, entries=[dict(id="a", tokens=ids["a"][:25], want=[3, 24])], end=[]),
             dict(step=1, entries=[dict(id="a", tokens=ids["a"][25:26], want=[0]), dict(id="b", tokens=ids["b"], want=[8])], end=["b"]),
             dict(step=2, entries=[dict(id="a", tokens=ids["a"][26:], want=[13])], end=["a"])]
    prog = Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    res = subprocess.run([sys.executable, str(prog), "--model", str(d), "--dtype", dtype, "--out", str(tmp_path),
                          "--max-tokens", "128", "--block-size", "4"], input="\n".join(map(json.dumps, lines)) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr[-2000:]
    assert [l for l in res.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    full = {k: plain.forward(v, w, cfg) for k, v in ids.items()}
    for step, wanted in ((0, [("a", 3), ("a", 24)]), (1, [("a", 25), ("b", 8)]), (2, [("a", 39)])):
        got = torch.from_numpy(np.fromfile(tmp_path / f"{step}.f32", dtype="<f4").reshape(len(wanted), cfg["vocab"]))
        check_logits(got, torch.stack([full[k][p] for k, p in wanted]), dtype, f"trace step {step}")


def test_command_line_writes_random_weights_and_generates(models, tmp_path):
    """bin/dinfer random-weights from a configuration that names the decay projection's inner size, then bin/dinfer
    generate on that folder and on a folder of the plain model's weights, where the greedy tokens are the plain
    model's wherever its choice is clear."""
    import subprocess
    import sys
    from pathlib import Path
    d, cfg, w, page = models["V1"]
    root = Path(__file__).resolve().parent.parent
    exe = [sys.executable, str(root / "bin" / "dinfer")]
    named = copy.deepcopy(cfg)
    for l in named["layers"]:
        if l["type"] == "parallel":
            l["mixer"]["right"]["decay_rank"] = 9
    (tmp_path / "config.json").write_text(json.dumps(named))
    p = subprocess.run(exe + ["random-weights", "--config", str(tmp_path / "config.json"), "--out", str(tmp_path / "m"), "--seed", "3"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    common = ["--dtype", "float32", "--max-model-len", "128", "--max-num-seqs", "2", "--num-blocks", "64", "--block-size", str(page),
              "--max-num-batched-tokens", "64", "--max-tokens", "8", "--temperature", "0", "--prompt-ids", "5,9,2", "--prompt-ids", "7"]
    p = subprocess.run(exe + ["generate", "--model", str(tmp_path / "m")] + common, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    recs = [json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")]
    assert [r["prompt_ids"] for r in recs] == [[5, 9, 2], [7]] and all(len(r["output_ids"]) == 8 for r in recs)
    p = subprocess.run(exe + ["generate", "--model", str(d)] + common, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    for r in (json.loads(l) for l in p.stdout.splitlines() if l.startswith("{")):
        ids = list(r["prompt_ids"])
        for tok in r["output_ids"]:
            logits = plain.forward(ids, w, cfg)[-1]
            top2 = logits.topk(2).values
            if (top2[0] - top2[1]).item() > 1e-3 * logits.std().item():
                assert tok == int(logits.argmax())
            ids.append(tok)
