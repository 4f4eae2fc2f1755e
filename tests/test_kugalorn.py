"""The plain Kugalorn implementation pinned by hand values that a plausible misreading fails, and the
configuration's refusals, declared tensors and caches.  No GPU."""
import math

import pytest
import torch

import kugalorn_util as ku
from plain import kugalorn_plain as plain

F64 = torch.float64


def test_norm_weight_is_stored_around_zero():
    x = torch.tensor([[3.0, -4.0]], dtype=F64)
    rms = math.sqrt(12.5 + 0.5)
    got = plain.offset_norm(x, torch.tensor([0.0, 1.0], dtype=F64), 0.5)
    assert torch.allclose(got, torch.tensor([[3.0 / rms, -8.0 / rms]], dtype=F64))          # (1 + w), eps inside the root
    assert torch.allclose(plain.plain_norm(x, torch.tensor([0.0, 1.0], dtype=F64), 0.5), torch.tensor([[0.0, -4.0 / rms]], dtype=F64))


def test_slopes_and_rotation_pairs():
    assert torch.allclose(plain.head_slopes(4), torch.tensor([0.25, 0.0625, 2.0 ** -6, 2.0 ** -8], dtype=F64))
    assert torch.allclose(plain.head_slopes(1), torch.tensor([2.0 ** -8], dtype=F64))
    # neighbours turn together (not the halves), by position * base^(-2i/dims); what lies beyond dims passes
    x = torch.tensor([[1.0, 0.0, 0.0, 2.0, 5.0, 7.0]], dtype=F64).repeat(2, 1)
    got = plain.rotate_pairs(x, torch.tensor([0, 3]), 100.0, 4)
    assert torch.equal(got[0], x[0])
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    want = torch.tensor([math.cos(a0), math.sin(a0), -2.0 * math.sin(a1), 2.0 * math.cos(a1), 5.0, 7.0], dtype=F64)
    assert torch.allclose(got[1], want)


def _attention_inputs(T, H, G, dk, dv, seed=0):
    g = torch.Generator().manual_seed(seed)
    d = H * dk + G * dk + G * dv
    eye = torch.eye(d, dtype=F64)
    W = {"q": eye[:H * dk], "k": eye[H * dk:(H + G) * dk], "v": eye[(H + G) * dk:], "o": torch.eye(H * dv, dtype=F64)}
    return torch.randn(T, d, generator=g, dtype=F64), W


def test_window_holds_the_token_and_size_minus_one_before_it():
    T, size = 9, 4
    x, W = _attention_inputs(T, 1, 1, 4, 3)
    m = dict(heads=1, kv_heads=1, dim=4, vdim=3, scale=0.5, mask={"size": size})
    base = plain.window_attention(x, W, m, 1e-6)
    for j, seen in ((T - 1 - size, False), (T - size, True), (T - 1, True)):
        y = x.clone()
        y[j, 8:] += 10.0                                         # the value of key j
        moved = (plain.window_attention(y, W, m, 1e-6)[T - 1] - base[T - 1]).abs().max() > 1e-6
        assert bool(moved) == seen, j


def test_scores_use_unit_queries_and_keys_and_lose_slope_times_distance():
    x, W = _attention_inputs(3, 2, 1, 2, 1, seed=1)
    m = dict(heads=2, kv_heads=1, dim=2, vdim=1, scale=0.7, mask={"size": 8})
    eps = 0.1
    got = plain.window_attention(x, W, m, eps)[2]
    unit = lambda v: v / math.sqrt(float((v * v).mean()) + eps)
    for h in range(2):
        q = unit(x[2, 2 * h:2 * h + 2])
        s = torch.stack([(q * unit(x[j, 4:6])).sum() * 0.7 - 2.0 ** (-8 * (h + 1) / 2) * (2 - j) for j in range(3)])
        p = torch.softmax(s, 0)
        assert torch.allclose(got[h], (p * x[:, 6]).sum())


def _latent_weights(m, d, seed=0):
    g = torch.Generator().manual_seed(seed)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    return {"q": r(H * (dk + dr), d), "dkv": r(rank + dr, d), "dkv.norm": 1 + 0.3 * r(rank), "uk": r(H * dk, rank) / 3,
            "uv": r(H * dv, rank) / 3, "g": r(H, d), "o": r(d, H * dv)}


def test_latent_attention_through_the_latent_space_is_the_same_function():
    """What an engine may compute instead of expanding keys and values: q' = [W_uk^T q_plain | q_rot] against the cached
    rows [c | k_rot], the rows' first `rank` channels as values, W_uv after the weighted sum."""
    m = ku.latent(3, 6, 4, 5, 10, 0.3, base=100.0, dims=2)["mixer"]
    d, T, eps = 12, 7, 1e-5
    W = _latent_weights(m, d)
    n = torch.randn(T, d, generator=torch.Generator().manual_seed(3), dtype=F64)
    want = plain.latent_attention(n, W, m, eps)
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (n @ W["q"].T).view(T, H, dk + dr)
    ckr = n @ W["dkv"].T
    rows = torch.cat([plain.plain_norm(ckr[:, :rank], W["dkv.norm"], eps), plain.rotate_pairs(ckr[:, rank:], pos, 100.0, 2)], 1)
    gate = torch.sigmoid(n @ W["g"].T)
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        ql = torch.cat([q[:, h, :dk] @ W["uk"][h * dk:(h + 1) * dk], plain.rotate_pairs(q[:, h, dk:], pos, 100.0, 2)], 1)
        s = (ql @ rows.T * m["scale"]).masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), -math.inf)
        out[:, h] = (torch.softmax(s, -1) @ rows[:, :rank]) @ W["uv"][h * dv:(h + 1) * dv].T * gate[:, h:h + 1]
    assert torch.allclose(out.reshape(T, -1) @ W["o"].T, want, atol=1e-10)


def test_latent_attention_is_causal_and_the_key_part_is_not_normed():
    m = ku.latent(2, 4, 2, 3, 6, 0.4)["mixer"]
    W = _latent_weights(m, 8, seed=1)
    n = torch.randn(5, 8, generator=torch.Generator().manual_seed(4), dtype=F64)
    base = plain.latent_attention(n, W, m, 1e-5)
    later = n.clone()
    later[4] += 1.0
    assert torch.equal(plain.latent_attention(later, W, m, 1e-5)[:4], base[:4])
    # scaling the rows of W_dkv that make the latent changes nothing but through eps; scaling the key part's rows does
    W2 = dict(W, dkv=torch.cat([W["dkv"][:6] * 3.0, W["dkv"][6:]]))
    assert torch.allclose(plain.latent_attention(n, W2, m, 0.0), plain.latent_attention(n, W, m, 0.0))
    W3 = dict(W, dkv=torch.cat([W["dkv"][:6], W["dkv"][6:] * 3.0]))
    assert not torch.allclose(plain.latent_attention(n, W3, m, 0.0), plain.latent_attention(n, W, m, 0.0))


def test_expert_clamps_the_gate_from_above_and_the_up_on_both_sides():
    one = torch.ones(1, 1, dtype=F64)
    f = lambda g, u, limit: float(plain.clamped_expert(one, torch.tensor([[g]], dtype=F64), torch.tensor([[u]], dtype=F64), one, limit))
    sw = lambda g: g / (1.0 + math.exp(-1.702 * g))
    assert f(0.5, 0.25, 1.0) == pytest.approx(sw(0.5) * 1.25)
    assert f(3.0, 0.25, 1.0) == pytest.approx(sw(1.0) * 1.25)            # gate capped
    assert f(-3.0, 0.25, 1.0) == pytest.approx(sw(-3.0) * 1.25)          # ... from above only
    assert f(0.5, 4.0, 1.0) == pytest.approx(sw(0.5) * 2.0)              # up capped
    assert f(0.5, -4.0, 1.0) == pytest.approx(0.0)                       # ... on both sides: (-1 + 1)


def test_router_adds_its_bias_and_weighs_the_chosen_alone():
    router = torch.tensor([[1.0], [2.0], [3.0], [0.0]], dtype=F64)
    bias = torch.tensor([0.0, 0.0, -5.0, 2.0], dtype=F64)
    ids, wts, z = plain.route(torch.ones(1, 1, dtype=F64), router, bias, 2)
    assert z.tolist() == [[1.0, 2.0, -2.0, 2.0]]
    assert ids.tolist() == [[1, 3]]                                       # a tie: the lower index first
    assert torch.allclose(wts, torch.tensor([[0.5, 0.5]], dtype=F64))     # the softmax of the two, not of the four


def test_streams_mix_from_the_old_values_and_the_matrix_is_from_to():
    xs = torch.tensor([[[1.0]], [[10.0]]], dtype=F64)                      # two streams, one token, one channel
    hc = {"in": torch.tensor([2.0, 0.5], dtype=F64), "out": torch.tensor([1.0, -1.0], dtype=F64),
          "mix": torch.tensor([[1.0, 3.0], [0.0, 1.0]], dtype=F64)}        # from stream 0 to stream 1: 3
    seen = []
    got = plain.hyper_step(xs, hc, lambda h: (seen.append(h), 100.0 * torch.ones_like(h))[1], torch.zeros(1, dtype=F64), 0.0)
    assert torch.allclose(seen[0], torch.ones(1, 1, dtype=F64))            # norm of u = 2 * 1 + 0.5 * 10 = 7 -> 1
    assert got[:, 0, 0].tolist() == [1.0 + 100.0, 3.0 * 1.0 + 10.0 - 100.0]


def test_run_order_and_every_pass_starts_from_the_streams_as_they_are():
    assert plain.layer_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert plain.layer_order({"layers": [0] * 3}) == [0, 1, 2]
    assert plain.layer_order({"layers": [0] * 3, "loop": {"start": 0, "stop": 3, "times": 1}}) == [0, 1, 2]
    raw = ku.CONFIGS["odd"]
    w = {k: v.to(F64) for k, v in ku.make_weights(raw, 0).items()}
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    outs = []
    logits = plain.forward(raw, w, toks, layer_outputs=outs)
    assert len(outs) == 7 and logits.shape == (8, raw["vocab"])
    unrolled = dict(raw, loop=None, layers=[raw["layers"][i] for i in plain.layer_order(raw)])
    w2 = {}
    for new, old in enumerate(plain.layer_order(raw)):
        w2.update({f"l{new}." + k: v for k, v in plain.sub(w, f"l{old}.").items()})
    w2.update({k: v for k, v in w.items() if not k.startswith("l")})
    assert torch.allclose(plain.forward(unrolled, w2, toks), logits)


# --------------------------------------------------------------------------- configuration
def test_configuration_reads_every_size_and_refuses_what_it_cannot_run():
    from tuff_amd.config.base import ConfigError
    from tuff_amd.models.registry import build_model, config_from_dict
    for name, raw in ku.CONFIGS.items():
        cfg = config_from_dict(raw)
        assert cfg.unknown_keys == [] and config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict(), name
        model = build_model(cfg)
        assert len(model.schedule) == len(plain.layer_order(raw)), name
    bad = [
        lambda r: r["layers"][0].update(type="conv"),
        lambda r: r["layers"][0]["mixer"].pop("scale"),
        lambda r: r["layers"][0]["mixer"].update(kv_heads=3),
        lambda r: r["layers"][0]["mixer"].update(mask={"size": 0}),
        lambda r: r["layers"][1]["mixer"]["rot"].update(dims=3),
        lambda r: r["layers"][1]["mixer"]["rot"].update(dims=64),
        lambda r: r["layers"][0]["mlp"]["router"].update(top=9),
        lambda r: r["layers"][0]["mlp"]["expert"].pop("limit"),
        lambda r: r["layers"][0]["mlp"].update(kind="dense"),
        lambda r: r.update(loop={"start": 2, "stop": 1, "times": 2}),
        lambda r: r.update(loop={"start": 0, "stop": 9, "times": 2}),
        lambda r: r.update(streams=0),
        lambda r: r["norm"].update(eps=0),
    ]
    import copy
    for i, spoil in enumerate(bad):
        raw = copy.deepcopy(ku.K_MIXED)
        spoil(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)
            pytest.fail(f"case {i} was accepted")


def test_declared_tensors_and_caches():
    from tuff_amd.cache.manager import CacheLayout
    from tuff_amd.models.registry import build_model, config_from_dict
    from tuff_amd.parts.base import PagedKV
    model = build_model(config_from_dict(ku.K_MIXED))
    decls = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert decls["l0.mix.q"] == (64, 64) and decls["l0.mix.v"] == (48, 64) and decls["l0.mix.o"] == (64, 96)
    assert decls["l1.mix.q"] == (48, 64) and decls["l1.mix.dkv"] == (40, 64) and decls["l1.mix.dkv.norm"] == (32,)
    assert decls["l1.mix.uk"] == (32, 32) and decls["l1.mix.uv"] == (48, 32) and decls["l1.mix.g"] == (2, 64)
    assert decls["l0.mlp.e3.gate"] == (40, 64) and decls["l0.mlp.router.b"] == (4,) and decls["l0.mlp.shared.down"] == (64, 24)
    assert decls["l0.hc1.mix"] == (2, 2) and decls["l0.hc2.in"] == (2,) and "l2.hc2.in" not in decls and "l2.norm2" not in decls
    assert "l3.mlp.shared.gate" not in decls
    # six runs (layers 1 and 2 twice), each with an entry of its own; a latent entry keeps one row a token, once
    # (36 channels: no multiple of 8) or a second time the way the matrix cores read values (40 channels)
    layout = CacheLayout.from_specs(model.cache_specs)
    assert len(layout.paged) == 6 and not layout.states
    assert sorted(layout.group_windows, key=str) == [20, 7, None]
    specs = list(layout.paged.values())
    assert specs.count(PagedKV(1, 40, None)) == 2 and specs.count(PagedKV(1, 36, None, value_dim=24, values_in_keys=True)) == 1
    assert layout.bytes_per_token(2) == 2 * (2 * (16 + 24) + 2 * (40 + 40) + 2 * (32 + 32) + 36)
    # without 'streams' the model has no such tensors and ordinary blocks
    plain_model = build_model(config_from_dict(ku.K_PLAIN))
    assert not any(".hc" in d.name for d in plain_model.weight_decls()) and plain_model.streams is None


def test_random_model_folder_round_trip(tmp_path):
    from tuff_amd.models.registry import config_from_dict, load_config
    from tuff_amd.weights.random_init import write_random_model
    from tuff_amd.weights.loader import Checkpoint
    cfg = config_from_dict(ku.K_MIXED)
    write_random_model(cfg, str(tmp_path), seed=3)
    assert load_config(str(tmp_path)).to_dict() == cfg.to_dict()
    from safetensors import safe_open
    with safe_open(str(tmp_path / "model.safetensors"), "pt") as f:
        mix, inn, norm = f.get_tensor("l0.hc1.mix").float(), f.get_tensor("l0.hc1.in").float(), f.get_tensor("l0.norm1").float()
    # the streams start near the plain residual sum: a unit mixing matrix, a mean as the read, norm weights around zero
    assert (mix - torch.eye(2)).abs().max() < 0.1 and (inn - 0.5).abs().max() < 0.1 and norm.abs().max() < 0.2
    assert set(Checkpoint(str(tmp_path)).names()) == {d.name for d in __import__("tuff_amd.models.registry", fromlist=["x"]).build_model(cfg).weight_decls()}
