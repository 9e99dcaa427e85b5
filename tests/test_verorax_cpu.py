"""Verorax without a GPU: the configuration and its refusals, the size that only a tensor's shape gives, run order and
tensor names of the model description, the caches its layers ask for, and the plain float64 model (plain_verorax.py)
pinned by library functions and hand-worked cases."""
import copy
import json
import math

import pytest
import torch

import plain_verorax as plain

F = torch.float64


def latent():
    return dict(type="latent_attention", mlp=dict(kind="dense", ff=40),
                mixer=dict(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=32, q_rank=20, scale=0.2, rot=dict(base=1000.0, dims=8)))


def differential():
    return dict(type="attention", mlp=None,
                mixer=dict(heads=4, kv_heads=2, dim=8, vdim=16, scale=0.35, diff=0.2, mask=dict(size=9)))


def parallel(rank=None):
    right = dict(heads=2, dim=16)
    if rank is not None:
        right["decay_rank"] = rank
    return dict(type="parallel", mlp=dict(kind="moe", expert=dict(ff=24), router=dict(experts=5, identity=2, top=2)),
                mixer=dict(left=dict(heads=4, kv_heads=1, dim=16, vdim=8, scale=0.25, mask=dict(size=7), rot=dict(base=500.0, dims=4)),
                           right=right, left_scale=0.7, right_scale=0.45))


def config(rank=6, **kw):
    cfg = dict(architecture="Verorax", vocab=96, width=64, norm=dict(eps=1e-5),
               layers=[latent(), parallel(rank), differential(), dict(copy.deepcopy(parallel(rank)), weights_of=1)])
    cfg.update(kw)
    return cfg


def parsed(cfg):
    from dinfer_amd.config.registry import architecture_of
    arch = architecture_of(cfg)
    return arch, arch.config_class.from_dict(cfg)


def test_config_round_trip_and_refusals():
    from dinfer_amd.config.base import ConfigError
    arch, cfg = parsed(config())
    assert arch.name == "Verorax" and cfg.vocab_size == 96 and cfg.hidden_size == 64
    assert type(cfg).from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    odd_rot = latent()
    odd_rot["mixer"]["rot"]["dims"] = 10                # more than the rotated part holds
    groups = differential()
    groups["mixer"]["kv_heads"] = 3
    far = parallel(6)
    far["mixer"]["left"]["rot"]["dims"] = 18
    many = parallel(6)
    many["mlp"]["router"]["top"] = 8
    bad = [dict(layers=[]), dict(norm=None), dict(layers=[dict(latent(), type="mamba")]), dict(layers=[odd_rot]),
           dict(layers=[groups]), dict(layers=[far]), dict(layers=[many]), dict(layers=[dict(latent(), mlp=dict(kind="glu"))]),
           dict(layers=[latent(), dict(latent(), weights_of=1)]), dict(layers=[latent(), dict(differential(), weights_of=0)]),
           dict(layers=[latent(), dict(latent(), weights_of=0), dict(latent(), weights_of=1)])]
    for change in bad:
        with pytest.raises(ConfigError):
            parsed(config(**change))
    with pytest.raises(ConfigError):                    # a layer on another's weights has a feed-forward if that one has
        parsed(config(layers=[latent(), dict(latent(), mlp=None, weights_of=0)]))
    with pytest.raises(ConfigError):                    # the decay projection's inner size is in no key and no tensor
        parsed(config(rank=None))


def test_the_size_that_only_a_tensor_gives(tmp_path):
    from dinfer_amd.config import load_config
    from dinfer_amd.weights.safetensors_io import write_safetensors
    cfg = config(rank=None)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    write_safetensors(tmp_path / "model.safetensors", plain.random_weights(cfg, 3, low=11), metadata={"format": "pt"})
    _, got = load_config(tmp_path)
    assert [l.mixer.right.decay_rank for l in got.layers if l.type == "parallel"] == [11, 11]
    cfg["layers"][1]["mixer"]["right"]["decay_rank"] = 4     # a file that names the size is taken at its word
    cfg["layers"][3]["mixer"]["right"]["decay_rank"] = 4
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    assert load_config(tmp_path)[1].layers[1].mixer.right.decay_rank == 4


def test_run_order_tensor_names_and_caches():
    from dinfer_amd.parts import DecoderModel
    arch, cfg = parsed(config(rank=6))
    spec = arch.build_spec(cfg)
    assert len(spec.layers) == 3 and [e.layer for e in spec.run] == [0, 1, 2, 1]
    assert spec.stream_dtype == "float32" and not spec.tie_embeddings
    m = DecoderModel(spec)
    exp, optional = m.expected_tensors()
    assert not optional
    shapes = plain.tensor_shapes(config(rank=6))
    assert {n: tuple(s.shape) for n, s in exp.items()} == {n: tuple(s) for n, s in shapes.items()}
    assert not any(n.startswith("l3.") for n in exp)


def test_a_layer_on_anothers_weights_with_constants_of_its_own():
    """Equal entries share one layer of the description; an entry that differs in a constant becomes a layer of its own
    under the same tensor names, and a size that does not fit those tensors is left to the check of the weights."""
    from dinfer_amd.parts import DecoderModel
    other = differential()
    other["mixer"]["mask"]["size"] = 4
    other["mixer"]["diff"] = 0.5
    cfg = config(layers=[differential(), dict(differential(), weights_of=0), dict(other, weights_of=0)])
    arch, c = parsed(cfg)
    spec = arch.build_spec(c)
    assert [e.layer for e in spec.run] == [0, 0, 1] and [l.prefix for l in spec.layers] == ["l0.", "l0."]
    assert spec.layers[1].mixer.params["window"] == 4 and spec.layers[0].mixer.params["window"] == 9
    exp, _ = DecoderModel(spec).expected_tensors()
    assert set(exp) == set(plain.tensor_shapes(cfg))


def test_token_shift_by_hand():
    h = torch.tensor([[2.0, 4.0], [6.0, 0.0], [1.0, 1.0]], dtype=F)
    out = plain.token_shift(h, torch.tensor([0.5, 1.0], dtype=F))
    assert out.tolist() == [[1.0, 0.0], [4.0, 4.0], [3.5, 0.0]]


def test_rotation_by_hand():
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]], dtype=F).repeat(2, 1, 1)       # two positions, one head of 6
    y = plain.rotate_halves(x, torch.tensor([0, 1]), dict(base=100.0, dims=4))
    assert torch.equal(y[0], x[0])                                                      # position 0 turns nothing
    f = [1.0, 100.0 ** -0.5]
    for i in (0, 1):                                                                    # entry i pairs with entry i + 2
        u, v = x[1, 0, i].item(), x[1, 0, i + 2].item()
        assert abs(y[1, 0, i].item() - (u * math.cos(f[i]) - v * math.sin(f[i]))) < 1e-12
        assert abs(y[1, 0, i + 2].item() - (v * math.cos(f[i]) + u * math.sin(f[i]))) < 1e-12
    assert y[1, 0, 4:].tolist() == [5.0, 6.0]


def test_windows_and_softmax_against_the_library():
    m = plain.visible(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True] and m[1].tolist() == [True, True, False, False, False, False]
    s = torch.randn(6, 6, dtype=F, generator=torch.Generator().manual_seed(1))
    p = plain.softmax_rows(s, m)
    assert torch.allclose(p[5, 3:], torch.softmax(s[5, 3:], -1)) and p[5, :3].abs().max().item() == 0.0
    z = torch.linspace(-3, 3, 13, dtype=F)
    assert torch.allclose(plain.gelu_tanh(z), torch.nn.functional.gelu(z, approximate="tanh"))
    assert torch.allclose(plain.silu(z), torch.nn.functional.silu(z))


def test_router_by_hand():
    """Three outputs, the last an identity expert: the correction moves the choice to the weaker score, the weight
    stays that score, and the identity expert hands the input on."""
    W = 2
    w = {"m.router": torch.tensor([[1.0, 0.0], [0.0, 1.0], [0.0, 0.0]], dtype=F), "m.correction": torch.tensor([0.0, 0.0, 0.8], dtype=F)}
    for e in range(2):
        w[f"m.e{e}.gate"] = torch.eye(W, dtype=F)
        w[f"m.e{e}.up"] = torch.eye(W, dtype=F) * (e + 1)
        w[f"m.e{e}.down"] = torch.eye(W, dtype=F)
    f = dict(kind="moe", expert=dict(ff=W), router=dict(experts=2, identity=1, top=1))
    h = torch.tensor([[2.0, 0.0]], dtype=F)
    s = torch.softmax(torch.tensor([2.0, 0.0, 0.0], dtype=F), -1)
    idx, share = plain.chosen_experts(h, w, "m", f)
    assert idx.tolist() == [[2]] and abs(share.item() - s[2].item()) < 1e-15       # 0.107 + 0.8 beats 0.787
    assert torch.allclose(plain.routed_ff(h, w, "m", f), s[2] * h)
    w["m.correction"] = torch.zeros(3, dtype=F)
    idx, share = plain.chosen_experts(h, w, "m", f)
    assert idx.tolist() == [[0]]
    want = s[0] * plain.silu(h) * h
    assert torch.allclose(plain.routed_ff(h, w, "m", f), want)


def test_delta_rule_by_hand():
    """One head of two channels, two tokens: the state after each token written out."""
    W = 2
    z = torch.zeros(2, 2, dtype=F)
    w = {"m.r": torch.eye(2, dtype=F), "m.k": torch.eye(2, dtype=F), "m.v": torch.eye(2, dtype=F) * 2, "m.g": z, "m.a": z,
         "m.a.b": torch.zeros(2, dtype=F), "m.w1": torch.zeros(1, 2, dtype=F), "m.w2": torch.zeros(2, 1, dtype=F),
         "m.w0": torch.zeros(2, dtype=F), "m.norm": torch.ones(2, dtype=F), "m.o": torch.eye(2, dtype=F)}
    h = torch.tensor([[1.0, 0.0], [1.0, 0.0]], dtype=F)
    decay = math.exp(-plain.DECAY_RATE * 0.5)
    # token 0: S = k v^T = [[2, 0], [0, 0]], o = S^T r = [2, 0]
    # token 1: u = [1, 0] (up to the eps under the root), a = 1/2: S_00 = decay * 2 - 0.5 * 2 + 2, o = [S_00, 0]
    s00 = decay * 2 - 0.5 * 2 / (1 + plain.UNIT_EPS) + 2
    out = plain.decayed_delta_rule(h, w, "m", dict(heads=1, dim=2), eps=0.0)
    # unit root mean square over the head's two values, times sigmoid(0) = 1/2
    assert torch.allclose(out[0], torch.tensor([math.sqrt(2) / 2, 0.0], dtype=F))
    assert torch.allclose(out[1], torch.tensor([math.sqrt(2) / 2, 0.0], dtype=F))
    S = torch.zeros(2, 2, dtype=F)
    S[0, 0] = 2.0
    u = torch.tensor([1.0, 0.0], dtype=F) / math.sqrt(1 + plain.UNIT_EPS)
    S1 = decay * S - torch.outer(0.5 * u, u @ S) + torch.outer(h[1], 2 * h[1])
    assert abs(S1[0, 0].item() - s00) < 1e-12


def test_differential_attention_of_one_key_and_lambda():
    """A window of one key: both maps return that key's value, so the head is (1 - lambda) v, normed."""
    cfg = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0, diff=0.25, mask=dict(size=1))
    g = torch.Generator().manual_seed(2)
    w = {"m." + n: torch.randn(s, dtype=F, generator=g) for n, s in
         (("q", (4, 3)), ("k", (4, 3)), ("v", (2, 3)), ("q.b", (4,)), ("k.b", (4,)), ("v.b", (2,)), ("lq1", (2,)), ("lk1", (2,)),
          ("lq2", (2,)), ("lk2", (2,)))}
    w["m.o"] = torch.eye(2, dtype=F)
    h = torch.randn(4, 3, dtype=F, generator=g)
    lam = math.exp(float(w["m.lq1"] @ w["m.lk1"])) - math.exp(float(w["m.lq2"] @ w["m.lk2"])) + 0.25
    v = h @ w["m.v"].T + w["m.v.b"]
    want = plain.rms_unit((1 - lam) * v, 1e-6) * 0.75
    assert torch.allclose(plain.differential_attention(h, w, "m", cfg, 1e-6), want)
