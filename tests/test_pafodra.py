"""Pafodra without a GPU: the configuration, the registry, the declared tensors and caches, and pins of
the plain implementation (hand values that a plausible misreading of a formula fails)."""
import copy
import math

import pytest
import torch

import pafodra_util as pu
from plain import pafodra_plain as plain


def cfg_of(raw):
    from tuff_amd.models.registry import config_from_dict
    return config_from_dict(raw)


def test_registered_by_its_one_name_spelling():
    from tuff_amd.config.pafodra import PafodraConfig
    from tuff_amd.models.registry import architectures
    assert "Pafodra" in architectures()
    cfg = cfg_of(pu.P_MIXED)
    assert isinstance(cfg, PafodraConfig) and cfg.vocab_size == 211 and cfg.hidden_size == 64
    assert cfg.owner(3) == 1 and cfg.owner(4) == 0 and cfg.owner(5) == 5
    chained = copy.deepcopy(pu.P_MIXED)
    chained["layers"].append(dict(chained["layers"][3], weights_of=3))          # through layer 3 to layer 1
    assert cfg_of(chained).owner(6) == 1
    assert cfg.rank(0, "w") == 8 and cfg.rank(5, "g") == 20
    again = cfg_of(cfg.to_dict())
    assert again.layers == cfg.layers and again.ranks == cfg.ranks


@pytest.mark.parametrize("edit, word", [
    (lambda r: r["layers"][0].update(type="mamba"), "type"),
    (lambda r: r["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda r: r["layers"][2]["mixer"].update(conv=0), "conv"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=9), "top"),
    (lambda r: r["layers"][3].update(weights_of=3), "weights_of"),
    (lambda r: r["layers"][3].update(weights_of=4), "which is a 'wkv' layer"),
    (lambda r: r["layers"][3].update(weights_of=0), "layer"),
    (lambda r: (r["layers"][3].update(weights_of=4), r["layers"][4].update(weights_of=3)), "weights_of"),
    (lambda r: r["norm"].update(eps=0), "eps"),
    (lambda r: r.pop("width"), "width"),
])
def test_bad_configurations_are_refused_in_words(edit, word):
    from tuff_amd.config.base import ConfigError
    raw = copy.deepcopy(pu.P_MIXED)
    edit(raw)
    with pytest.raises(ConfigError, match=word):
        cfg_of(raw)


def test_declared_tensors_and_caches():
    from tuff_amd.models.registry import build_model
    from tuff_amd.parts.base import FixedState, PagedKV
    model = build_model(cfg_of(pu.P_MIXED))
    shapes = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert not any(n.startswith(("l3.", "l4.")) for n in shapes)              # layers 3 and 4 have no tensors of their own
    assert shapes["l0.mix.w1"] == (8, 64) and shapes["l0.mix.w2"] == (32, 8) and shapes["l0.mix.u"] == (2, 16)
    assert shapes["l1.mix.q"] == (64, 64) and shapes["l1.mix.v"] == (48, 64) and shapes["l1.mix.o"] == (64, 96)
    assert shapes["l1.mix.sink"] == (4,) and shapes["l1.mlp.shared.sg"] == (1, 64) and shapes["l1.mlp.e3.down"] == (64, 40)
    assert shapes["l2.mix.q.conv"] == (32, 3) and shapes["l2.mix.v.conv"] == (32, 3) and shapes["l2.mix.norm"] == (8,)
    assert shapes["l2.mix.a2"] == (64, 16) and shapes["l2.mix.g2"] == (32, 8) and shapes["l2.mix.b"] == (4, 64)
    assert "l5.mlp.shared.up" not in shapes and shapes["l0.norm1.alpha"] == ()
    assert [r.block for r in model.schedule] == [0, 1, 2, 1, 0, 3]
    specs = model.cache_specs
    assert specs[1] == PagedKV(2, 16, None, value_dim=24) and specs[3] == specs[1]          # a cache each
    assert specs[(0, 0)] == FixedState((64,)) and specs[(4, 1)] == FixedState((2, 16, 16))
    assert specs[(2, 0)] == FixedState((2, 96)) and specs[(2, 1)] == FixedState((4, 16, 8))
    assert specs[(5, 0)] == FixedState((1, 2 * 48 + 80))
    assert model.graph_safe() and model.records_portions()


def test_ranks_come_from_the_checkpoints_shapes(tmp_path):
    from tuff_amd.models.registry import load_config
    folder = pu.write_folder(pu.P_WIDE, pu.make_weights(pu.P_WIDE, 1), str(tmp_path / "m"))
    cfg = load_config(folder)
    assert cfg.ranks == {"l0": {"a": 5, "g": 9}, "l1": {"w": 3}}


# ------------------------------------------------------------------ pins of the plain implementation
def test_dyt_by_hand():
    x = torch.tensor([[0.5, -2.0]], dtype=torch.float64)
    y = plain.dyt(x, torch.tensor([2.0, 3.0]), torch.tensor([0.1, -0.1]), torch.tensor(0.5))
    assert torch.allclose(y, torch.tensor([[2 * math.tanh(0.25) + 0.1, 3 * math.tanh(-1.0) - 0.1]], dtype=torch.float64))


def test_causal_conv_last_tap_is_the_current_token():
    x = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    y = plain.causal_conv(x, torch.tensor([[2.0, 3.0, 5.0]], dtype=torch.float64))
    assert y[:, 0].tolist() == [5.0, 53.0, 532.0]


def test_sink_counts_once_unscaled_and_has_no_value():
    # one token, one head: the weight of the only key is e^s / (e^s + e^sink), s = q.k * scale
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=0.5)
    eye = torch.eye(2, dtype=torch.float64)
    W = {"q": eye, "k": eye, "v": eye, "o": eye, "sink": torch.tensor([0.7], dtype=torch.float64)}
    n = torch.tensor([[2.0, 1.0]], dtype=torch.float64)
    s = 5.0 * 0.5
    want = n * math.exp(s) / (math.exp(s) + math.exp(0.7))
    assert torch.allclose(plain.sink_attention(n, W, "", m), want)
    # a second token sees both keys; the first still sees only its own
    n2 = torch.tensor([[2.0, 1.0], [0.0, 3.0]], dtype=torch.float64)
    out = plain.sink_attention(n2, W, "", m)
    assert torch.allclose(out[0], want[0])
    s0, s1 = 3.0 * 0.5, 9.0 * 0.5
    den = math.exp(s0) + math.exp(s1) + math.exp(0.7)
    assert torch.allclose(out[1], (math.exp(s0) * n2[0] + math.exp(s1) * n2[1]) / den)


def _wkv_weights(d, H, D, rank=2):
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    W = {"mu." + s: z(d) for s in "rkvgw"}
    eye = torch.eye(H * D, d, dtype=torch.float64)
    W.update(r=eye.clone(), k=eye.clone(), v=eye.clone(), g=eye.clone(), w1=z(rank, d), w2=z(H * D, rank), w0=z(H * D),
             u=z(H, D), norm=torch.ones(H * D, dtype=torch.float64), o=torch.eye(d, H * D, dtype=torch.float64))
    return W


def test_wkv_bonus_for_the_current_token_only_and_decay_after_the_read():
    d = H_D = 2
    W = _wkv_weights(d, 1, 2)
    W["u"] = torch.tensor([[0.5, 0.25]], dtype=torch.float64)
    W["w0"] = torch.tensor([0.0, math.log(2.0)], dtype=torch.float64)          # decays e^-1 and e^-2
    n = torch.tensor([[1.0, 2.0], [3.0, 1.0]], dtype=torch.float64)
    m = dict(heads=1, dim=2)
    # token 0: o = (u k r summed) v = (0.5 + 0.25 * 4) * [1, 2];  S = k v^T
    o0 = 1.5 * n[0]
    # token 1: o = S^T r + bonus v, S = outer(n0, n0) not yet decayed
    S = torch.outer(n[0], n[0])
    o1 = S.T @ n[1] + (0.5 * 9 + 0.25 * 1) * n[1]
    o = torch.stack([o0, o1])
    want = plain.unit_rms(o, 1e-5) * plain.silu(n)
    assert torch.allclose(plain.wkv(n, W, m, 1e-5), want)
    # the third token reads the state decayed once after each write
    n3 = torch.cat([n, torch.tensor([[1.0, 1.0]], dtype=torch.float64)])
    S2 = torch.diag(torch.tensor([math.exp(-1.0), math.exp(-2.0)], dtype=torch.float64)) @ S + torch.outer(n[1], n[1])
    o2 = S2.T @ n3[2] + 0.75 * n3[2]
    got = plain.wkv(n3, W, m, 1e-5)[2]
    assert torch.allclose(got, plain.unit_rms(o2[None], 1e-5)[0] * plain.silu(n3[2]))


def test_wkv_blends_with_the_token_before_and_zeros_at_the_start():
    W = _wkv_weights(2, 1, 2)
    W["mu.k"] = torch.tensor([1.0, 0.5], dtype=torch.float64)          # k reads h' in channel 0, the mean in channel 1
    W["u"] = torch.ones(1, 2, dtype=torch.float64)
    n = torch.tensor([[4.0, 2.0], [1.0, 6.0]], dtype=torch.float64)
    out = plain.wkv(n[:1], W, dict(heads=1, dim=2), 1e-5)
    k0 = torch.tensor([0.0, 1.0], dtype=torch.float64)                 # zeros stand before the first token
    o0 = (k0 * n[0]).sum() * n[0]
    assert torch.allclose(out[0], plain.unit_rms(o0[None], 1e-5)[0] * plain.silu(n[0]))


def test_delta_rule_first_tokens_by_hand():
    d, H, D, Dv = 2, 1, 2, 2
    eye = torch.eye(2, dtype=torch.float64)
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    one_tap = torch.tensor([[0.0, 1.0]] * 2, dtype=torch.float64)
    W = {"q": eye, "k": eye, "v": eye, "q.conv": one_tap, "k.conv": one_tap, "v.conv": one_tap, "b": z(1, 2),
         "a1": z(1, 2), "a2": z(2, 1), "dt_bias": z(2), "A_log": z(1), "g1": z(1, 2), "g2": z(2, 1),
         "norm": torch.ones(2, dtype=torch.float64), "o": eye}
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, conv=2)
    n = torch.tensor([[1.0, 2.0], [2.0, -1.0]], dtype=torch.float64)
    a = plain.silu(n)
    unit = lambda x: x / torch.sqrt((x * x).sum() + 1e-6)
    k0, k1 = unit(a[0]), unit(a[1])
    q0, q1 = k0 / math.sqrt(2.0), k1 / math.sqrt(2.0)
    beta, g = 0.5, math.exp(-math.log(2.0))                            # sigmoid(0); exp(-e^0 softplus(0))
    S = torch.outer(k0, beta * a[0])                                   # from zero: the error is v itself
    o0 = S.T @ q0
    S = g * S
    S = S + torch.outer(k1, beta * (a[1] - S.T @ k1))
    o1 = S.T @ q1                                                       # the read sees the token's own write
    want = plain.unit_rms(torch.stack([o0, o1]), 1e-5) * 0.5           # gate sigmoid(0)
    assert torch.allclose(plain.channel_delta(n, W, m, 1e-5), want)


def test_moe_scales_the_input_keeps_scores_and_gates_the_shared_expert():
    d = 2
    t64 = lambda v: torch.tensor(v, dtype=torch.float64)
    W = {"router": t64([[1.0, 0.0], [0.0, 1.0], [-1.0, -1.0]]),
         "e0.up": t64([[1.0, 0.0]]), "e0.down": t64([[1.0], [0.0]]),
         "e1.up": t64([[0.0, 1.0]]), "e1.down": t64([[0.0], [1.0]]),
         "e2.up": t64([[1.0, 1.0]]), "e2.down": t64([[1.0], [1.0]]),
         "shared.up": t64([[1.0, 1.0]]), "shared.down": t64([[2.0], [0.0]]), "shared.sg": t64([[0.5, 0.0]])}
    n = t64([[2.0, 1.0]])
    sig = lambda v: 1.0 / (1.0 + math.exp(-v))
    spec = {"router": {"experts": 3, "top": 2}, "shared": {"ff": 1}}
    # experts 0 and 1 are chosen with weights sigmoid(2), sigmoid(1), not renormalised; relu squared of the scaled input
    want = t64([[(sig(2.0) * 2.0) ** 2, (sig(1.0) * 1.0) ** 2]])
    want[0, 0] += sig(1.0) * 2.0 * 9.0                                 # shared: sigmoid(0.5 * 2) * down(relu(3)^2)
    assert torch.allclose(plain.moe_ff(n, W, spec), want)
    spec1 = {"router": {"experts": 3, "top": 1}}
    assert torch.allclose(plain.moe_ff(n, W, spec1), t64([[(sig(2.0) * 2.0) ** 2, 0.0]]))


def test_dense_feed_forward_by_hand():
    t64 = lambda v: torch.tensor(v, dtype=torch.float64)
    W = {"gate": t64([[1.0, 0.0]]), "gate.b": t64([0.5]), "up": t64([[0.0, 2.0]]), "up.b": t64([-1.0]),
         "down": t64([[1.0], [3.0]]), "down.b": t64([0.25, -0.25])}
    z = 1.5
    gelu = 0.5 * z * (1.0 + math.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))
    a = gelu * (2.0 * 2.0 - 1.0)
    assert torch.allclose(plain.dense_ff(t64([[1.0, 2.0]]), W), t64([[a + 0.25, 3 * a - 0.25]]))


def test_layer_is_parallel_and_shared_tensors_run_twice():
    raw = pu.config(16, 23, [pu.layer(pu.attn(1, 1, 8, 8, 0.3), pu.dense(24)), pu.layer(pu.attn(1, 1, 8, 8, 0.3), pu.dense(24), weights_of=0)])
    w = pu.make_weights(raw, 3)
    toks = [3, 7, 1, 22, 5]
    layers = []
    plain.forward(raw, w, toks, layers_out=layers)
    W = {k: v.double() for k, v in w.items()}
    x0 = W["embed"][torch.tensor(toks)] * raw["embedding"]["scale"]
    n = plain.dyt(x0, W["l0.norm1"], W["l0.norm1.b"], W["l0.norm1.alpha"])
    both = plain.sink_attention(n, plain.sub(W, "l0.mix."), "", raw["layers"][0]["mixer"]) + plain.dense_ff(n, plain.sub(W, "l0.mlp."))
    assert torch.allclose(layers[0], x0 + both)                         # both sublayers read the same normed rows
    n1 = plain.dyt(layers[0], W["l0.norm1"], W["l0.norm1.b"], W["l0.norm1.alpha"])
    again = plain.sink_attention(n1, plain.sub(W, "l0.mix."), "", raw["layers"][0]["mixer"]) + plain.dense_ff(n1, plain.sub(W, "l0.mlp."))
    assert torch.allclose(layers[1], layers[0] + again)
