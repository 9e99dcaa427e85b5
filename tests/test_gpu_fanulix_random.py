"""Fanulix models drawn at random (widths, head counts and sizes, layer order, decays, rotated entries, temperature
steps, taps, groups, experts, streams, pages), each replayed in mixed batches and in portions against the plain float64
model, in both dtypes: nothing in the engine may rest on the sizes of one model."""
import json
import random

import pytest
import torch

import plain_fanulix as plain
from test_gpu_fanulix import check_logits, cut, mixed_schedule, replay, tokens_for

pytestmark = pytest.mark.gpu
SEEDS = range(8)


def draw_config(seed):
    rng = random.Random(seed)
    pick = rng.choice

    def parallel():
        kv, dim = pick([1, 2, 3]), pick([8, 12, 16, 24, 32, 40, 64])
        rh, rd = pick([1, 2, 3, 4]), pick([8, 12, 16, 20, 32, 48, 64])
        return dict(
            left=dict(heads=kv * pick([1, 2, 4]), kv_heads=kv, dim=dim, vdim=pick([dim, dim, 8, 16, 20, 32, 48]),
                      scale=round(rng.uniform(0.5, 1.5) * dim ** -0.5, 4),
                      q_temp=dict(coef=pick([0.0, 0.25, 0.5, 1.0]), every=pick([1, 3, 8, 16, 64, 1000]))),
            right=dict(heads=rh, dim=rd, vdim=pick([8, 12, 16, 24, 40, 64]),
                       decay=[pick([0.5, 0.875, 0.9375, 0.99, 0.999, 1.0]) for _ in range(rh)],
                       rot=dict(base=pick([100.0, 10000.0, 1000000.0]), dims=pick([d for d in range(0, rd + 1, 2)]))),
            left_scale=round(rng.uniform(0.2, 1.2), 3), right_scale=round(rng.uniform(0.2, 1.2), 3))

    def state_space():
        groups = pick([1, 2, 3])
        heads = groups * pick([1, 2, 4])
        vdim = pick([8, 12, 16, 24, 32])
        return dict(heads=heads, vdim=vdim, state=pick([8, 16, 24, 32, 64]), groups=groups, conv=pick([1, 2, 3, 4, 5]),
                    norm_groups=pick([g for g in (1, 2, 3, 4, heads) if (heads * vdim) % g == 0]))

    def routed():
        experts = pick([2, 3, 5, 8, 12, 16])
        return dict(kind="moe", router=dict(experts=experts, top=rng.randint(1, min(experts, 4))), expert=dict(ff=pick([8, 12, 24, 40])),
                    shared=None if rng.random() < 0.25 else dict(ff=pick([8, 20, 32, 48])))

    layers = []
    for _ in range(rng.randint(2, 5)):
        kind = pick(["parallel", "parallel", "mamba2"])
        layers.append(dict(type=kind, mixer=parallel() if kind == "parallel" else state_space(),
                           mlp=None if rng.random() < 0.2 else routed()))
    cfg = dict(architecture="Fanulix", vocab=rng.randint(50, 150), width=pick([32, 40, 48, 64, 80, 104]),
               logit_scale=pick([0.5, 1.0, 2.0]), norm=dict(eps=pick([1e-6, 1e-5, 1e-3])), layers=layers)
    streams = pick([None, 1, 2, 3, 4, 5])
    if streams is not None:
        cfg["streams"] = streams
    return cfg, pick([4, 8, 16])


def compare_rows(rows, cfg, w, toks, dtype, what, runner=None):
    """32-bit: every row close to the plain model. bfloat16: through models this narrow a token whose best experts score
    nearly alike may be sent to another one by a rounding (with one expert a token that is a different feed-forward), and
    what it then adds to the recurrent states stays with the tokens behind it. So the rows are held to the plain model as
    a whole (a wrong key, a lost state or a sink left out moves most rows by more), and, sharply, to the engine's own
    bfloat16 logits of each request alone in one step: cuts, batches, pages and slots must not show beyond rounding."""
    assert rows
    errs, own = [], []
    for rid in sorted({k[0] for k in rows}):
        ids = toks[rid.split("#")[0]]
        want = plain.forward(cfg, w, ids)
        pos = sorted(p for (r, p) in rows if r == rid)
        got = torch.stack([rows[(rid, p)] for p in pos])
        if dtype == "float32":
            check_logits(got, want[pos], dtype, f"{what} request {rid}")
            continue
        sd = want[pos].std(dim=-1, keepdim=True)
        errs.append(((got - want[pos]).abs() / sd).max(dim=-1).values)
        alone = replay(runner, [([("alone", ids, pos)], ["alone"])])
        alone = torch.stack([alone[("alone", p)] for p in pos])
        own.append(((got - alone).abs() / sd).max(dim=-1).values)
    if errs:
        e, o = torch.cat(errs).sort().values, torch.cat(own).sort().values
        assert e[len(e) // 2] < 0.3 and e[-1] < 6.0, \
            f"{what}: bf16 rows off by {e[len(e) // 2]:.3f} (median), {e[int(len(e) * 0.9)]:.3f} (90 %), {e[-1]:.3f} (worst) row-sigmas"
        assert o[len(o) // 2] < 0.03 and o[int(len(o) * 0.9)] < 0.3, \
            f"{what}: bf16 rows differ from the same request alone by {o[len(o) // 2]:.3f} (median), {o[int(len(o) * 0.9)]:.3f} (90 %)"


@pytest.fixture(scope="module")
def drawn(tmp_path_factory):
    from dinfer_amd.weights.safetensors_io import write_safetensors
    out = {}
    for seed in SEEDS:
        cfg, page = draw_config(200 + seed)
        d = tmp_path_factory.mktemp(f"fanulix_r{seed}")
        w = plain.random_weights(cfg, seed)
        (d / "config.json").write_text(json.dumps(cfg))
        write_safetensors(d / "model.safetensors", {k: v.to(torch.bfloat16) for k, v in w.items()}, metadata={"format": "pt"})
        out[seed] = (d, cfg, w, page)
    return out


def runner_for(drawn, seed, dtype, num_blocks, max_len=128):
    from dinfer_amd.config import EngineOptions
    from dinfer_amd.engine.runner import ModelRunner
    d, _, _, page = drawn[seed]
    opt = EngineOptions(dtype=dtype, max_model_len=max_len, max_num_seqs=4, max_num_batched_tokens=256, block_size=page,
                        num_blocks=num_blocks, max_logits_rows=256, decode_exempt_from_budget=False, hip_graph=True)
    return ModelRunner.from_dir(d, opt)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", SEEDS)
def test_drawn_model_in_mixed_batches_and_portions(drawn, seed, dtype):
    _, cfg, w, page = drawn[seed]
    toks, steps = mixed_schedule(cfg, seed)
    r = runner_for(drawn, seed, dtype, num_blocks=4 * (96 // page) + 4, max_len=96)
    compare_rows(replay(r, steps), cfg, w, toks, dtype, f"drawn model {seed}, mixed", r)
    ids = tokens_for(cfg, 90, seed)
    parts = cut(ids, [13, 2, 1, 1, 1, 30, 5])
    rows = replay(r, [([("x", p, list(range(len(p))))], ["x"] if i == len(parts) - 1 else []) for i, p in enumerate(parts)])
    compare_rows(rows, cfg, w, {"x": ids}, dtype, f"drawn model {seed}, portions", r)


def test_drawn_configurations_differ():
    """The draw covers both mixers, layers without a feed-forward, models without `streams` and with several."""
    cfgs = [draw_config(200 + s)[0] for s in SEEDS]
    kinds = {l["type"] for c in cfgs for l in c["layers"]}
    assert kinds == {"parallel", "mamba2"}
    assert any(l["mlp"] is None for c in cfgs for l in c["layers"]) and any("streams" not in c for c in cfgs)
    assert any((c.get("streams") or 1) > 1 for c in cfgs)
