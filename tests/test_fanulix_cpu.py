"""Fanulix without a GPU: the configuration and its refusals, the model description (parts, tensor names, caches), and
the plain float64 model (plain_fanulix.py) pinned by library functions and hand-worked cases."""
import json
import math

import pytest
import torch

import plain_fanulix as plain

F = torch.float64


def par(**kw):
    m = dict(left=dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.25, q_temp=dict(coef=0.5, every=8)),
             right=dict(heads=2, dim=16, vdim=8, decay=[0.9, 0.995], rot=dict(base=1000.0, dims=8)), left_scale=0.7, right_scale=0.45)
    m.update(kw)
    return dict(type="parallel", mixer=m, mlp=dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=24), shared=dict(ff=16)))


def ssm(**kw):
    m = dict(heads=4, vdim=8, state=16, groups=2, conv=3, norm_groups=2)
    m.update(kw)
    return dict(type="mamba2", mixer=m, mlp=None)


def config(**kw):
    cfg = dict(architecture="Fanulix", vocab=96, width=64, logit_scale=1.5, streams=2, norm=dict(eps=1e-5), layers=[par(), ssm(), par()])
    cfg.update(kw)
    return cfg


def parsed(cfg):
    from dinfer_amd.config.registry import architecture_of
    arch = architecture_of(cfg)
    return arch, arch.config_class.from_dict(cfg)


def test_config_round_trip_and_refusals():
    from dinfer_amd.config.base import ConfigError
    arch, cfg = parsed(config())
    assert arch.name == "Fanulix" and cfg.vocab_size == 96 and cfg.hidden_size == 64 and cfg.streams == 2
    assert type(cfg).from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    no_streams = config()
    del no_streams["streams"]
    assert parsed(no_streams)[1].streams is None
    bad_right = par()
    bad_right["mixer"]["right"]["decay"] = [0.9]                  # one decay a head
    odd_rot = par()
    odd_rot["mixer"]["right"]["rot"]["dims"] = 7
    wide_rot = par()
    wide_rot["mixer"]["right"]["rot"]["dims"] = 18
    bad_heads = par()
    bad_heads["mixer"]["left"]["kv_heads"] = 3
    dense = par()
    dense["mlp"] = dict(kind="dense", ff=8)
    greedy = par()
    greedy["mlp"]["router"]["top"] = 6
    bad = [dict(layers=[bad_right]), dict(layers=[odd_rot]), dict(layers=[wide_rot]), dict(layers=[bad_heads]), dict(layers=[dense]),
           dict(layers=[greedy]), dict(layers=[dict(par(), type="attention")]), dict(layers=[ssm(groups=3)]),
           dict(layers=[ssm(norm_groups=5)]), dict(layers=[]), dict(norm=None), dict(streams=0)]
    for change in bad:
        with pytest.raises(ConfigError):
            parsed(config(**change))


def test_parts_tensor_names_and_caches():
    from dinfer_amd.parts.model import DecoderModel, expected_tensors
    arch, cfg = parsed(config())
    spec = arch.build_spec(cfg)
    exp, optional = expected_tensors(spec)
    want = plain.tensor_shapes(config())
    assert {k: tuple(v.shape) for k, v in exp.items()} == {k: tuple(v) for k, v in want.items()}
    assert optional == {"head"} and spec.tie_embeddings and spec.streams == 2 and spec.stream_dtype == "float32"
    assert [l.block.kind for l in spec.layers] == ["streams"] * 3
    assert [l.mixer.kind for l in spec.layers] == ["joined", "state_space", "joined"]
    assert [l.feed_forward.kind for l in spec.layers] == ["moe", "none", "moe"]
    model = DecoderModel(spec)
    needs = model.cache_needs()
    # a parallel layer: pages of keys and values of their own sizes, and a matrix a retention head
    left, right = needs[0].members["left"], needs[0].members["right"]
    assert (left.kv_heads, left.head_dim, left.v_dim, left.window) == (2, 16, 24, None)
    assert (right.heads, right.dim, right.vdim, right.channels, right.taps) == (2, 16, 8, 0, 1)
    assert not needs[0].recomputable and needs[0].group_key() is not None
    # a state-space layer: no pages; a matrix a head and the convolution's last inputs
    assert needs[1].group_key() is None
    assert (needs[1].heads, needs[1].dim, needs[1].vdim, needs[1].channels, needs[1].taps) == (4, 16, 8, 4 * 8 + 2 * 2 * 16, 3)
    # without `streams`: the plain pre-norm residual, no stream weights in the file
    plain_cfg = config()
    del plain_cfg["streams"]
    spec = arch.build_spec(parsed(plain_cfg)[1])
    assert spec.streams == 1 and [l.block.kind for l in spec.layers] == ["prenorm"] * 3
    assert not any(".hc" in k for k in expected_tensors(spec)[0])


def test_random_model_folder_reads_back(tmp_path):
    from dinfer_amd.config import load_config
    from dinfer_amd.weights import write_random_model
    from dinfer_amd.weights.safetensors_io import SafetensorsDir
    _, cfg = parsed(config())
    write_random_model(cfg, tmp_path, seed=3)
    arch, back = load_config(tmp_path)
    assert back == cfg
    files = SafetensorsDir(tmp_path)
    assert {k: tuple(files.info(k).shape) for k in files.names()} == {k: tuple(v) for k, v in plain.tensor_shapes(config()).items()}


# ---- the plain model itself ---------------------------------------------------------------------------------------
def test_plain_small_functions():
    x = torch.randn(5, 12, dtype=F)
    assert torch.allclose(plain.gelu_erf(x), torch.nn.functional.gelu(x))
    assert torch.allclose(plain.silu(x), torch.nn.functional.silu(x))
    assert torch.allclose(plain.softplus(x * 10), torch.nn.functional.softplus(x * 10))
    w, b = torch.randn(12, dtype=F), torch.randn(12, dtype=F)
    assert torch.allclose(plain.layer_norm(x, w, b, 1e-5), torch.nn.functional.layer_norm(x, (12,), w, b, 1e-5))
    assert torch.allclose(plain.rms_unit(x, 0.0).pow(2).mean(-1), torch.ones(5, dtype=F))


def test_plain_softmax_with_a_sink_of_score_zero():
    s = torch.tensor([[0.0, math.log(2.0), -50.0]], dtype=F)
    p = plain.softmax_plus_one(s, torch.tensor([[True, True, False]]))
    assert torch.allclose(p, torch.tensor([[0.25, 0.5, 0.0]], dtype=F))          # 1 + 1 + 2 in the denominator
    big = plain.softmax_plus_one(torch.tensor([[800.0]], dtype=F), torch.tensor([[True]]))
    assert abs(big.item() - 1.0) < 1e-12                                         # no overflow
    assert plain.query_temperature(torch.tensor([0, 6, 7, 15, 16]), 0.5, 8).tolist() == pytest.approx(
        [1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3), 1 + 0.5 * math.log(3)])


def test_plain_rotation_and_recurrence():
    x = torch.randn(6, 2, 10, dtype=F)
    pos = torch.arange(6) * 7
    y = plain.rotate_half(x, pos, 100.0, 6)
    assert torch.equal(y[..., 6:], x[..., 6:])                                   # entries beyond `dims` pass unchanged
    z = torch.complex(x[..., :3], x[..., 3:6]) * torch.polar(torch.ones(6, 3, dtype=F),
                                                             pos.to(F)[:, None] * torch.tensor([100.0 ** (-2 * i / 6) for i in range(3)], dtype=F))[:, None]
    assert torch.allclose(y[..., :3], z.real) and torch.allclose(y[..., 3:6], z.imag)
    # a recurrence without decay is causal linear attention; with a decay the weights are its powers
    q, k, v = torch.randn(7, 4, dtype=F), torch.randn(7, 4, dtype=F), torch.randn(7, 3, dtype=F)
    a = torch.full((7,), 0.8, dtype=F)
    o = plain.decayed_recurrence(q, k, v, a)
    w = torch.tril(0.8 ** (torch.arange(7)[:, None] - torch.arange(7)[None, :]).clamp(min=0).to(F))
    assert torch.allclose(o, ((q @ k.T) * w) @ v)
    gain = torch.rand(7, dtype=F)
    assert torch.allclose(plain.decayed_recurrence(q, k, v, a, gain), ((q @ k.T) * w * gain[None, :]) @ v)


def test_plain_convolution_routing_and_streams():
    x, taps, bias = torch.randn(9, 5, dtype=F), torch.randn(5, 3, dtype=F), torch.randn(5, dtype=F)
    lib = torch.nn.functional.conv1d(x.T[None], taps[:, None, :], bias, padding=2, groups=5)[0, :, :9].T
    assert torch.allclose(plain.causal_conv(x, taps, bias), lib)
    h, router = torch.randn(4, 6, dtype=F), torch.randn(5, 6, dtype=F)
    idx, share = plain.route(h, router, 2)
    assert torch.allclose(share.sum(-1), torch.ones(4, dtype=F))
    z = h @ router.T
    assert torch.equal(idx, z.topk(2).indices)
    assert torch.allclose(share, torch.softmax(z.gather(1, idx), -1))           # the softmax over the chosen logits
    xs = torch.randn(3, 2, 4, dtype=F)
    mix = torch.randn(3, 3, dtype=F)
    out = plain.streams_write(xs, torch.zeros(2, 4, dtype=F), mix, torch.zeros(3, dtype=F))
    assert torch.allclose(out[1], mix[0, 1] * xs[0] + mix[1, 1] * xs[1] + mix[2, 1] * xs[2])     # indexed [from, to]
    # a model of several equal streams with unit weights is the plain residual model
    cfg = config(streams=1, layers=[ssm()])
    w = plain.random_weights(cfg, 1)
    w["l0.hc1.in"], w["l0.hc1.out"], w["l0.hc1.mix"] = (torch.ones(1, dtype=F), torch.ones(1, dtype=F), torch.ones(1, 1, dtype=F))
    plain_cfg = dict(cfg)
    del plain_cfg["streams"]
    ids = [3, 9, 27, 81, 5]
    assert torch.allclose(plain.forward(cfg, w, ids), plain.forward(plain_cfg, w, ids))
