"""The plain Loluzen implementation pinned by hand values that a plausible misreading fails, and the
configuration's refusals, declared tensors and caches.  No GPU."""
import copy
import math

import pytest
import torch

import loluzen_util as lu
from plain import loluzen_plain as plain

F64 = torch.float64
t64 = lambda *v: torch.tensor(v, dtype=F64)


def test_norm_weight_is_stored_around_zero_and_the_plain_one_is_not():
    x = t64([3.0, -4.0])
    rms = math.sqrt(12.5 + 0.5)
    assert torch.allclose(plain.offset_norm(x, t64(0.0, 1.0), 0.5), t64([3.0 / rms, -8.0 / rms]))        # (1 + w), eps inside the root
    assert torch.allclose(plain.plain_norm(x, t64(0.0, 1.0), 0.5), t64([0.0, -4.0 / rms]))


def test_frequencies_fall_into_three_ranges_by_wavelength():
    # original 64, low 1, high 4: wavelengths below 16 stay, above 64 are divided, between the two a share stays
    base, dims = 1000.0, 8
    plainf = [base ** (-2.0 * i / dims) for i in range(4)]
    got = plain.scaled_frequencies(base, dims, dict(factor=8.0, low=1.0, high=4.0, original=64))
    waves = [2 * math.pi / f for f in plainf]
    assert waves[0] < 16 < waves[1] < 64 < waves[2]                   # one in each range, the last two above
    assert got[0] == plainf[0]
    s = (64 / waves[1] - 1.0) / 3.0
    assert got[1] == pytest.approx((1 - s) * plainf[1] / 8.0 + s * plainf[1])
    assert got[2] == pytest.approx(plainf[2] / 8.0) and got[3] == pytest.approx(plainf[3] / 8.0)
    assert torch.equal(plain.scaled_frequencies(base, dims), t64(*plainf))


def test_rotation_turns_neighbours_over_the_first_channels_only():
    x = t64([1.0, 0.0, 0.0, 2.0, 5.0, 7.0]).repeat(2, 1)
    fr = t64(1.0, 0.1)
    got = plain.rotate_pairs(x, torch.tensor([0, 3]), fr)
    assert torch.equal(got[0], x[0])
    want = t64(math.cos(3.0), math.sin(3.0), -2.0 * math.sin(0.3), 2.0 * math.cos(0.3), 5.0, 7.0)
    assert torch.allclose(got[1], want)


def test_convolution_ends_at_the_token_and_its_last_tap_is_the_token_itself():
    u = t64([1.0], [10.0], [100.0], [1000.0])
    taps = t64([2.0, 3.0, 5.0])                                # [C = 1, K = 3]
    got = plain.short_convolution(u, taps)
    assert got[:, 0].tolist() == [5.0, 50.0 + 3.0, 500.0 + 30.0 + 2.0, 5000.0 + 300.0 + 20.0]


def _identity_attention(T, H, G, dk, dv, seed=0):
    g = torch.Generator().manual_seed(seed)
    d = H * dk + G * dk + G * dv
    eye = torch.eye(d, dtype=F64)
    W = {"q": eye[:H * dk], "k": eye[H * dk:(H + G) * dk], "v": eye[(H + G) * dk:], "o": torch.eye(H * dv, dtype=F64),
         "q.b": torch.zeros(H * dk, dtype=F64), "k.b": torch.zeros(G * dk, dtype=F64), "v.b": torch.zeros(G * dv, dtype=F64),
         "g": torch.zeros(H, d, dtype=F64), "r1": torch.zeros(H, dtype=F64), "r2": torch.zeros(H, dtype=F64),
         "talk": torch.eye(H, dtype=F64)}
    return torch.randn(T, d, generator=g, dtype=F64), W


def test_distance_penalty_is_a_logarithm_taken_off_the_scaled_score():
    x, W = _identity_attention(4, 2, 1, 2, 1)
    m = dict(heads=2, kv_heads=1, dim=2, vdim=1, scale=0.7)
    W["r1"], W["r2"] = t64(0.5, 2.0), t64(3.0, 0.25)
    got = plain.biased_talking_attention(x, W, m)[3]
    for h in range(2):
        s = torch.stack([(x[3, 2 * h:2 * h + 2] * x[j, 4:6]).sum() * 0.7 - W["r1"][h] * math.log(1 + float(W["r2"][h]) * (3 - j))
                         for j in range(4)])
        assert torch.allclose(got[h], 0.5 * (torch.softmax(s, 0) * x[:, 6]).sum())         # (the gate's logit is 0)


def test_heads_weights_are_mixed_after_the_softmax_and_meet_their_own_values():
    """talk[h, g] weighs head g's softmax in head h's mixture; head h then reads the values of its own kv head."""
    T = 5
    x, W = _identity_attention(T, 2, 2, 3, 2, seed=2)
    m = dict(heads=2, kv_heads=2, dim=3, vdim=2, scale=0.9)
    W["talk"] = t64([0.25, 2.0], [0.0, 1.0])
    got = plain.biased_talking_attention(x, W, m).view(T, 2, 2)
    q, k, v = x[:, :6].view(T, 2, 3), x[:, 6:12].view(T, 2, 3), x[:, 12:].view(T, 2, 2)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    p = [torch.softmax((q[:, h] @ k[:, h].T * 0.9).masked_fill(~causal, -math.inf), -1) for h in range(2)]
    assert torch.allclose(got[:, 0], 0.5 * (0.25 * p[0] + 2.0 * p[1]) @ v[:, 0])       # head 0: both softmaxes, its own values
    assert torch.allclose(got[:, 1], 0.5 * p[1] @ v[:, 1])
    # mixing the scores before the softmax, or the outputs after the values, are other functions
    mixed_outputs = 0.5 * (0.25 * p[0] @ v[:, 0] + 2.0 * p[1] @ v[:, 1])
    assert not torch.allclose(got[:, 0], mixed_outputs)


def test_bias_enters_the_projection_and_the_gate_reads_the_mixers_input():
    x, W = _identity_attention(3, 1, 1, 2, 2, seed=3)
    m = dict(heads=1, kv_heads=1, dim=2, vdim=2, scale=1.0)
    base = plain.biased_talking_attention(x, W, m)
    W2 = dict(W)
    W2["v.b"] = t64(1.0, -2.0)
    assert torch.allclose(plain.biased_talking_attention(x, W2, m), base + 0.5 * t64(1.0, -2.0))     # softmax weights sum to 1
    W3 = dict(W)
    W3["g"] = torch.zeros(1, 6, dtype=F64)
    W3["g"][0, 0] = 1.0
    assert torch.allclose(plain.biased_talking_attention(x, W3, m), base * 2.0 * torch.sigmoid(x[:, 0:1]))


def test_forget_gate_also_sets_how_much_is_written():
    """One head, one key channel, one value channel: S_t = f S_(t-1) + (1 - f) v_t, o_t = S_t silu(q_t); the gate never
    falls below `lower`."""
    m = dict(heads=1, dim=1, vdim=1)
    W = {"q": t64([1.0, 0.0, 0.0]), "f": t64([0.0, 1.0, 0.0]), "v": t64([0.0, 0.0, 1.0]), "f.b": t64(0.5), "lower": t64(0.2),
         "norm": t64(1.0), "o": t64([1.0])}
    n = t64([1.0, -30.0, 2.0], [2.0, 0.0, -1.0], [-1.0, 30.0, 5.0])
    f = [0.2 + 0.8 / (1 + math.exp(-(z + 0.5))) for z in (-30.0, 0.0, 30.0)]
    assert f[0] == pytest.approx(0.2) and f[2] == pytest.approx(1.0)
    S, want = 0.0, []
    silu = lambda z: z / (1 + math.exp(-z))
    for t in range(3):
        S = f[t] * S + (1 - f[t]) * float(n[t, 2])
        want.append(S * silu(float(n[t, 0])))
    out, state = plain.forget_gate_recurrence(n, W, m, 0.0)
    # (the norm over one channel leaves the sign: compare before it through the state, and the sign after)
    assert float(state[0, 0, 0]) == pytest.approx(S)
    assert [float(v) for v in torch.sign(out[:, 0])] == [math.copysign(1.0, w) for w in want]
    out2, state2 = plain.forget_gate_recurrence(n[2:], W, m, 0.0, state=plain.forget_gate_recurrence(n[:2], W, m, 0.0)[1])
    assert torch.allclose(state2, state) and torch.allclose(out2, out[2:])


def test_recurrence_output_is_normed_per_head_with_one_weight():
    m = dict(heads=2, dim=2, vdim=3)
    g = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    W = {"q": r(4, 6), "f": r(4, 6), "v": r(6, 6), "f.b": r(4), "lower": torch.rand(4, generator=g, dtype=F64), "norm": r(3),
         "o": torch.eye(6, dtype=F64)}
    out, _ = plain.forget_gate_recurrence(r(4, 6), W, m, 0.0)
    heads = out.view(4, 2, 3) / W["norm"]
    assert torch.allclose((heads * heads).mean(-1), torch.ones(4, 2, dtype=F64))


def test_pair_is_half_the_sum_of_the_two_normed_outputs():
    raw = lu.ONLY["pair"]
    w = {k: v.to(F64) for k, v in lu.make_weights(raw, 1).items()}
    L = {k[len("l0.mix."):]: v for k, v in w.items() if k.startswith("l0.mix.")}
    n = torch.randn(6, raw["width"], generator=torch.Generator().manual_seed(1), dtype=F64)
    m = raw["layers"][0]["mixer"]
    left = plain.biased_talking_attention(n, {k[5:]: v for k, v in L.items() if k.startswith("left.") and k != "left.out"}, m["left"])
    right, _ = plain.forget_gate_recurrence(n, {k[6:]: v for k, v in L.items() if k.startswith("right.") and k != "right.out"}, m["right"], 1e-5)
    want = 0.5 * (plain.plain_norm(left, L["left.out"], 1e-5) + plain.plain_norm(right, L["right.out"], 1e-5))
    assert torch.allclose(plain.pair_mixer(n, L, m, 1e-5), want)


def test_convolution_comes_before_the_norm_and_the_norm_before_the_rotation():
    raw = lu.ONLY["attention"]
    m = raw["layers"][0]["mixer"]
    w = {k[len("l0.mix."):]: v.to(F64) for k, v in lu.make_weights(raw, 2).items() if k.startswith("l0.mix.")}
    n = torch.randn(7, raw["width"], generator=torch.Generator().manual_seed(2), dtype=F64)
    T, H, G, dk, dv = 7, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    fr = plain.scaled_frequencies(m["rot"]["base"], m["rot"]["dims"], m["rot"]["scaling"])
    pos = torch.arange(T)
    q = plain.short_convolution(n @ w["q"].T, w["q.conv"]).view(T, H, dk)
    k = plain.short_convolution(n @ w["k"].T, w["k.conv"]).view(T, G, dk)
    v = plain.short_convolution(n @ w["v"].T, w["v.conv"]).view(T, G, dv)
    q = plain.rotate_pairs(plain.plain_norm(q, w["q.norm"], 1e-5), pos, fr)
    k = plain.rotate_pairs(plain.plain_norm(k, w["k.norm"], 1e-5), pos, fr)
    gate = torch.sigmoid(n @ w["g"].T)
    out = torch.zeros(T, H, dv, dtype=F64)
    causal = torch.tril(torch.ones(T, T, dtype=torch.bool))
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T * m["scale"]).masked_fill(~causal, -math.inf)
        out[:, h] = torch.softmax(s, -1) @ v[:, h // (H // G)] * gate[:, h:h + 1]
    assert torch.allclose(out.reshape(T, -1) @ w["o"].T, plain.conv_rotary_attention(n, w, m, 1e-5))
    # causal: a later token moves nothing before it
    later = n.clone()
    later[5] += 1.0
    assert torch.equal(plain.conv_rotary_attention(later, w, m, 1e-5)[:5], plain.conv_rotary_attention(n, w, m, 1e-5)[:5])


def test_feed_forward_squares_the_relu_and_has_both_biases():
    W = {"up": t64([1.0], [-1.0]), "up.b": t64(0.5, 0.25), "down": t64([2.0, 3.0]), "down.b": t64(-1.0)}
    assert plain.squared_relu_mlp(t64([1.0]), W).tolist() == [[2.0 * 1.5 ** 2 - 1.0]]
    assert plain.squared_relu_mlp(t64([-2.0]), W).tolist() == [[3.0 * 2.25 ** 2 - 1.0]]


def test_run_order_and_the_embedding_joins_again_before_every_later_pass():
    order = plain.run_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}})
    assert order == [(0, False), (1, False), (2, False), (1, True), (2, False), (1, True), (2, False), (3, False), (4, False)]
    assert plain.run_order({"layers": [0] * 2}) == [(0, False), (1, False)]
    assert plain.run_order({"layers": [0] * 2, "loop": {"start": 0, "stop": 2, "times": 1}}) == [(0, False), (1, False)]
    raw = lu.ONLY["loop"]
    w = lu.make_weights(raw, 0)
    toks = [3, 1, 4, 1, 5, 9, 2, 6]
    outs = []
    logits = plain.forward(raw, w, toks, layers_out=outs)
    assert len(outs) == 6 and logits.shape == (8, raw["vocab"])
    # unrolled with copies of the tensors, the embedding added by hand: the same function
    W = {k: v.to(F64) for k, v in w.items()}
    x0 = W["embed"][torch.tensor(toks)] * raw["embedding"]["scale"]
    once = dict(raw, loop=None)
    x = x0.clone()
    for p in range(3):
        if p:
            x = x + x0
        for i in range(2):
            one = dict(once, layers=[raw["layers"][i]])
            w1 = {"l0." + k[3:]: v for k, v in w.items() if k.startswith(f"l{i}.")}
            w1.update(embed=torch.eye(raw["width"]), head=torch.eye(raw["width"]), **{"final.norm": torch.zeros(raw["width"])})
            ys = []
            # (a one-layer model fed the stream through an identity embedding cannot be built from token ids: run the layer's
            # own functions instead)
            n = plain.offset_norm(x, W[f"l{i}.norm1"], 1e-5)
            L = {k[len(f"l{i}.mix."):]: v for k, v in W.items() if k.startswith(f"l{i}.mix.")}
            layer = raw["layers"][i]
            y = plain.pair_mixer(n, L, layer["mixer"], 1e-5) if layer["type"] == "parallel" else plain.conv_rotary_attention(n, L, layer["mixer"], 1e-5)
            x = x + raw["residual_mult"] * plain.offset_norm(y, W[f"l{i}.norm1b"], 1e-5)
            if layer["mlp"] is not None:
                M = {k[len(f"l{i}.mlp."):]: v for k, v in W.items() if k.startswith(f"l{i}.mlp.")}
                x = x + raw["residual_mult"] * plain.offset_norm(plain.squared_relu_mlp(plain.offset_norm(x, W[f"l{i}.norm2"], 1e-5), M),
                                                                 W[f"l{i}.norm2b"], 1e-5)
            assert torch.allclose(x, outs[2 * p + i]), (p, i)
    assert torch.allclose(plain.offset_norm(x, W["final.norm"], 1e-5) @ W["head"].T, logits)


# --------------------------------------------------------------------------- configuration
def test_configuration_reads_every_size_and_refuses_what_it_cannot_run():
    from tuff_amd.config.base import ConfigError
    from tuff_amd.models.registry import build_model, config_from_dict
    for name, raw in lu.CONFIGS.items():
        cfg = config_from_dict(raw)
        assert cfg.unknown_keys == [] and config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict(), name
        model = build_model(cfg)
        assert [(r.block, r.reinject) for r in model.schedule] == plain.run_order(raw), name
    bad = [
        lambda r: r["layers"][0].update(type="conv"),
        lambda r: r["layers"][0]["mixer"]["left"].pop("scale"),
        lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3),
        lambda r: r["layers"][0]["mixer"].pop("right"),
        lambda r: r["layers"][0]["mixer"]["right"].update(dim=0),
        lambda r: r["layers"][1]["mixer"]["rot"].update(dims=3),
        lambda r: r["layers"][1]["mixer"]["rot"].update(dims=64),
        lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].pop("original"),
        lambda r: r["layers"][1]["mixer"]["rot"]["scaling"].update(high=1.0),
        lambda r: r["layers"][1]["mixer"].update(conv=0),
        lambda r: r["layers"][0]["mlp"].update(kind="experts"),
        lambda r: r["layers"][0]["mlp"].pop("ff"),
        lambda r: r.update(loop={"start": 2, "stop": 1, "times": 2}),
        lambda r: r.update(loop={"start": 0, "stop": 9, "times": 2}),
        lambda r: r.update(loop={"start": 0, "stop": 2, "times": 0}),
        lambda r: r["norm"].update(eps=0),
        lambda r: r.update(layers=[]),
        lambda r: r["embedding"].pop("scale"),
    ]
    for i, spoil in enumerate(bad):
        raw = copy.deepcopy(lu.L_MIXED)
        spoil(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)
            pytest.fail(f"case {i} was accepted")


def test_declared_tensors_and_caches():
    from tuff_amd.cache.manager import CacheLayout
    from tuff_amd.models.registry import build_model, config_from_dict
    from tuff_amd.parts.base import FixedState, PagedKV
    model = build_model(config_from_dict(lu.L_MIXED))
    decls = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert decls["l0.mix.left.q"] == (64, 64) and decls["l0.mix.left.k"] == (32, 64) and decls["l0.mix.left.q.b"] == (64,)
    assert decls["l0.mix.left.talk"] == (4, 4) and decls["l0.mix.left.r1"] == (4,) and decls["l0.mix.left.g"] == (4, 64)
    assert decls["l0.mix.right.q"] == (32, 64) and decls["l0.mix.right.v"] == (48, 64) and decls["l0.mix.right.lower"] == (32,)
    assert decls["l0.mix.right.norm"] == (24,) and decls["l0.mix.left.out"] == (64,) and decls["l0.mix.right.o"] == (64, 48)
    assert decls["l1.mix.q"] == (96, 64) and decls["l1.mix.v"] == (32, 64) and decls["l1.mix.q.conv"] == (96, 3)
    assert decls["l1.mix.v.conv"] == (32, 3) and decls["l1.mix.k.norm"] == (24,) and decls["l1.mix.o"] == (64, 64)
    assert decls["l0.mlp.up.b"] == (40,) and decls["l0.mlp.down.b"] == (64,) and "l2.mlp.up" not in decls and "l2.norm2" not in decls
    assert decls["final.norm"] == (64,) and decls["head"] == (211, 64)
    # six runs (layers 1 and 2 twice), each with cache and state of its own: a pair keeps keys and values and a state a
    # head, a convolution's attention its last taps - 1 projected rows and keys and values
    layout = CacheLayout.from_specs(model.cache_specs)
    specs = list(layout.paged.values())
    assert len(specs) == 6 and specs.count(PagedKV(2, 24, None, value_dim=16)) == 2 and specs.count(PagedKV(1, 32, None, value_dim=8)) == 2
    states = list(layout.states.values())
    assert states.count(FixedState((2, 16, 24))) == 1 and states.count(FixedState((3, 8, 16))) == 2
    assert states.count(FixedState((2, 96 + 48 + 32))) == 2 and states.count(FixedState((1, 32 + 32 + 32))) == 1
    # one tap and no taps keep no rows
    odd = CacheLayout.from_specs(build_model(config_from_dict(lu.L_ODD)).cache_specs)
    assert sum(isinstance(s, FixedState) and len(s.shape) == 2 for s in odd.states.values()) == 0


def test_random_model_folder_round_trip(tmp_path):
    from tuff_amd.models.registry import build_model, config_from_dict, load_config
    from tuff_amd.weights.loader import Checkpoint
    from tuff_amd.weights.random_init import write_random_model
    cfg = config_from_dict(lu.L_WIDE)
    write_random_model(cfg, str(tmp_path), seed=3)
    assert load_config(str(tmp_path)).to_dict() == cfg.to_dict()
    assert set(Checkpoint(str(tmp_path)).names()) == {d.name for d in build_model(cfg).weight_decls()}
    from safetensors import safe_open
    with safe_open(str(tmp_path / "model.safetensors"), "pt") as f:
        lower, talk = f.get_tensor("l1.mix.right.lower").float(), f.get_tensor("l1.mix.left.talk").float()
    assert 0 < lower.min() and lower.max() < 1 and (talk - torch.eye(6)).abs().max() < 0.2
