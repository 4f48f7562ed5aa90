"""The plain Kinelix implementation pinned by hand values that a plausible misreading fails, and the
configuration's refusals, declared tensors and caches.  No GPU."""
import copy
import math

import pytest
import torch

import kinelix_util as xu
from plain import kinelix_plain as plain

F64 = torch.float64
t64 = lambda v: torch.tensor(v, dtype=F64)


def test_layer_norm_takes_the_mean_off_has_no_bias_and_eps_inside_the_root():
    x = t64([[1.0, 3.0, 5.0, 7.0]])
    got = plain.layer_norm(x, t64([1.0, 2.0, 0.0, -1.0]), 0.5)
    sd = math.sqrt(5.0 + 0.5)                                   # deviations -3 -1 1 3: variance 5 (not 20 / 3)
    assert torch.allclose(got, t64([[-3.0 / sd, -2.0 / sd, 0.0, -3.0 / sd]]))
    assert torch.allclose(plain.layer_norm(x + 100.0, t64([1.0, 2.0, 0.0, -1.0]), 0.5), got)       # a shift of the row does nothing


def test_convolution_last_tap_is_the_tokens_own_zeros_stand_before_and_the_bias_is_inside_the_activation():
    x = t64([[1.0], [10.0], [100.0]])
    taps = t64([[3.0, 2.0, 1.0]])
    assert torch.equal(plain.causal_conv(x, taps), t64([[1.0], [12.0], [123.0]]))
    assert torch.equal(plain.causal_conv(x, taps, t64([0.5])), t64([[1.5], [12.5], [123.5]]))


def _mamba_weights(H, P, N, G, K, seed=0, norm_groups=1):
    """A mamba2 mixer whose input projection picks columns: a row of the input is [z | x | B | C | dt]."""
    inner = H * P
    width = 2 * inner + 2 * G * N + H
    g = torch.Generator().manual_seed(seed)
    conv = torch.zeros(inner + 2 * G * N, K, dtype=F64)
    conv[:, -1] = 1.0                                              # the convolution passes the token itself
    W = {"in": torch.eye(width, dtype=F64), "conv": conv, "conv.b": torch.zeros(inner + 2 * G * N, dtype=F64),
         "dt_bias": torch.randn(H, generator=g, dtype=F64), "A_log": torch.randn(H, generator=g, dtype=F64),
         "D": torch.randn(H, generator=g, dtype=F64), "norm": torch.ones(inner, dtype=F64), "o": torch.eye(inner, dtype=F64)}
    m = dict(heads=H, vdim=P, state=N, groups=G, norm_groups=norm_groups, conv=K)
    return W, m, width


def test_mamba2_by_hand_one_channel():
    """One head, one state channel, one value channel, two tokens: the decay is exp(-exp(A_log) dt) with dt behind a
    softplus, the write is dt B x, the read sees the token's own write, D x joins, the gate comes before the norm."""
    W, m, width = _mamba_weights(1, 1, 1, 1, 2)
    z, x, B, C, dt = [0.3, -0.8], [0.5, 2.0], [1.5, -0.7], [0.4, 1.1], [0.2, -0.3]
    n = t64([[z[t], x[t], B[t], C[t], dt[t]] for t in range(2)])
    silu = lambda v: v / (1.0 + math.exp(-v))
    xs, Bs, Cs = [silu(v) for v in x], [silu(v) for v in B], [silu(v) for v in C]
    dts = [math.log1p(math.exp(v + float(W["dt_bias"][0]))) for v in dt]
    A, D = math.exp(float(W["A_log"][0])), float(W["D"][0])
    S0 = dts[0] * Bs[0] * xs[0]
    y0 = S0 * Cs[0] + D * xs[0]
    S1 = math.exp(-A * dts[1]) * S0 + dts[1] * Bs[1] * xs[1]
    y1 = S1 * Cs[1] + D * xs[1]
    eps = 0.25
    want = [(y * silu(g)) / math.sqrt((y * silu(g)) ** 2 + eps) for y, g in ((y0, z[0]), (y1, z[1]))]
    got = plain.mamba2(n, W, m, eps)
    assert torch.allclose(got[:, 0], t64(want))


def test_mamba2_heads_read_their_groups_rows_and_the_norm_runs_in_parts():
    H, P, N, G = 4, 2, 3, 2
    W, m, width = _mamba_weights(H, P, N, G, 1, seed=1, norm_groups=2)
    g = torch.Generator().manual_seed(2)
    n = torch.randn(5, width, generator=g, dtype=F64)
    base = plain.mamba2(n, W, m, 1e-3)
    inner = H * P
    other = n.clone()
    other[:, 2 * inner + N:2 * inner + 2 * N] += 1.0               # B of group 1: heads 2 and 3 alone move ...
    moved = (plain.mamba2(other, W, m, 1e-3) - base).abs().sum(0).view(H, P).sum(1)
    assert moved[0] == 0 and moved[1] == 0 and moved[2] > 0 and moved[3] > 0
    big = n.clone()
    big[:, inner:inner + 1] *= 50.0                               # ... and a large x in head 0 shrinks its half of the norm only
    change = (plain.mamba2(big, W, m, 1e-3) - base).abs().sum(0)
    assert change[:inner // 2].min() > 0 and change[inner // 2:].max() == 0


def _delta_weights(H, Hk, D, Dv, seed=0):
    Cq, Cv = Hk * D, H * Dv
    width = 2 * Cq + 2 * Cv + 2 * H
    eye = torch.eye(width, dtype=F64)
    g = torch.Generator().manual_seed(seed)
    one = lambda c: torch.ones(c, 1, dtype=F64)
    W = {"q": eye[:Cq], "k": eye[Cq:2 * Cq], "v": eye[2 * Cq:2 * Cq + Cv], "g": eye[2 * Cq + Cv:2 * Cq + 2 * Cv],
         "b": eye[2 * Cq + 2 * Cv:2 * Cq + 2 * Cv + H], "a": eye[2 * Cq + 2 * Cv + H:],
         "q.conv": one(Cq), "k.conv": one(Cq), "v.conv": one(Cv), "A_log": torch.randn(H, generator=g, dtype=F64),
         "dt_bias": torch.randn(H, generator=g, dtype=F64), "norm": torch.ones(Dv, dtype=F64), "o": torch.eye(Cv, dtype=F64)}
    return W, dict(heads=H, kv_heads=Hk, dim=D, vdim=Dv, conv=1), width


def test_delta_rule_by_hand_decay_then_error_then_write_then_read():
    """One head, keys of one channel (a unit key is +-1), values of one channel, two tokens."""
    W, m, width = _delta_weights(1, 1, 1, 1)
    silu = lambda v: v / (1.0 + math.exp(-v))
    q, k, v, gate, b, a = [2.0, 3.0], [1.0, 2.0], [0.7, -1.2], [0.4, 0.9], [0.3, -0.6], [0.1, 0.5]
    n = t64([[q[t], k[t], v[t], gate[t], b[t], a[t]] for t in range(2)])
    unit = lambda x: x / math.sqrt(x * x + 1e-6)
    A, bias = math.exp(float(W["A_log"][0])), float(W["dt_bias"][0])
    S, outs = 0.0, []
    for t in range(2):
        qn, kn, vs = unit(silu(q[t])), unit(silu(k[t])), silu(v[t])            # dim 1: q also times 1^-1/2
        dec = math.exp(-A * math.log1p(math.exp(a[t] + bias)))
        beta = 1.0 / (1.0 + math.exp(-b[t]))
        S = dec * S
        S = S + kn * beta * (vs - S * kn)
        outs.append(S * qn)
    eps = 0.5
    want = [o / math.sqrt(o * o + eps) * silu(gt) for o, gt in zip(outs, gate)]
    assert torch.allclose(plain.gated_delta(n, W, m, eps)[:, 0], t64(want))


def test_delta_rule_has_one_decay_a_head_and_value_heads_share_the_keys_of_their_group():
    H, Hk, D, Dv = 4, 2, 3, 2
    W, m, width = _delta_weights(H, Hk, D, Dv, seed=3)
    g = torch.Generator().manual_seed(4)
    n = torch.randn(6, width, generator=g, dtype=F64)
    base = plain.gated_delta(n, W, m, 1e-3)
    other = n.clone()
    other[:3, D:2 * D] += 2.0                                    # q of key head 1, early tokens: value heads 2 and 3 alone move
    moved = (plain.gated_delta(other, W, m, 1e-3) - base).abs().sum(0).view(H, Dv).sum(1)
    assert moved[0] == 0 and moved[1] == 0 and moved[2] > 0 and moved[3] > 0
    decay = n.clone()
    decay[:, -H] += 3.0                                          # a of head 0
    moved = (plain.gated_delta(decay, W, m, 1e-3) - base).abs().sum(0).view(H, Dv).sum(1)
    assert moved[0] > 0 and moved[1:].max() == 0


def _latent_weights(H, dk, dv, rank, sink):
    g = torch.Generator().manual_seed(H + dk)
    r = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    width = H * dk + rank
    eye = torch.eye(width, dtype=F64)
    return {"q": eye[:H * dk], "dkv": eye[H * dk:], "dkv.norm": 1.0 + 0.3 * r(rank), "uk": r(H * dk, rank), "uv": r(H * dv, rank),
            "sink": t64(sink), "o": torch.eye(H * dv, dtype=F64)}, dict(heads=H, dim=dk, vdim=dv, kv_rank=rank, scale=0.4), width


def test_sink_counts_once_unscaled_without_a_value_and_attention_is_causal():
    W, m, width = _latent_weights(1, 2, 3, 2, [math.log(3.0)])
    T = 4
    n = torch.zeros(T, width, dtype=F64)
    n[:, 2:] = torch.randn(T, 2, generator=torch.Generator().manual_seed(1), dtype=F64)
    c = plain.latent_rows(n, W, 1e-5)
    # zero queries: every score is 0, so the weights are 1 / (keys seen + exp(sink)) = 1 / (i + 1 + 3)
    v = (c @ W["uv"].T)
    got = plain.latent_attention(n, c, W, m)
    for i in range(T):
        assert torch.allclose(got[i], v[:i + 1].sum(0) / (i + 1 + 3.0))
    # a later token's row changes nothing before it
    n2 = n.clone()
    n2[3, 2:] += 1.0
    c2 = plain.latent_rows(n2, W, 1e-5)
    assert torch.equal(plain.latent_attention(n2, c2, W, m)[:3], got[:3])


def test_latent_rows_are_normed_with_a_plain_weight_and_scores_are_scaled():
    W, m, width = _latent_weights(2, 3, 2, 4, [-30.0, -30.0])       # sinks that hold nothing
    n = torch.randn(3, width, generator=torch.Generator().manual_seed(2), dtype=F64)
    c = plain.latent_rows(n, W, 0.1)
    raw = n[:, 6:]
    assert torch.allclose(c, raw / torch.sqrt((raw * raw).mean(-1, keepdim=True) + 0.1) * W["dkv.norm"])
    got = plain.latent_attention(n, c, W, m)[2]
    for h in range(2):
        k = c @ W["uk"][3 * h:3 * h + 3].T
        s = (k @ n[2, 3 * h:3 * h + 3]) * 0.4
        p = torch.softmax(s, 0)
        assert torch.allclose(got[2 * h:2 * h + 2], p @ (c @ W["uv"][2 * h:2 * h + 2].T), atol=1e-10)


def test_a_layer_reads_the_rows_of_the_layer_it_names_with_matrices_of_its_own():
    raw = xu.ONLY["latent_shared"]
    w = {k: v.double() for k, v in xu.make_weights(raw, 0).items()}
    toks = [3, 9, 27, 81, 5]
    seen = []
    base = plain.forward(raw, w, toks, on_layer=lambda i, x: seen.append(x.clone()))
    # the second layer has no narrow projection of its own ...
    assert "l1.mix.dkv" not in w and "l1.mix.uk" in w and "l1.mix.uv" in w
    # ... and sees the first layer's rows: with the first layer's own matrices silenced (its output gone), a change of
    # its narrow projection still moves the second layer
    w2 = dict(w)
    w2["l0.ls1"] = torch.zeros_like(w["l0.ls1"])
    a = plain.forward(raw, w2, toks)
    w3 = dict(w2)
    w3["l0.mix.dkv"] = w["l0.mix.dkv"].flip(0)
    assert (plain.forward(raw, w3, toks) - a).abs().max() > 1e-6


def _route_spec(E, top, count, keep, scale):
    return {"router": {"experts": E, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


def test_router_correction_enters_the_choice_only_and_weights_are_scores_times_scale():
    n = t64([[1.0, 0.0]])
    router = t64([[2.0, 0.0], [1.0, 0.0], [0.0, 0.0], [-1.0, 0.0]])
    s = torch.sigmoid(t64([2.0, 1.0, 0.0, -1.0]))
    W = {"router": router, "correction": t64([0.0, 0.0, 0.0, 1.0])}
    ids, wts = plain.route(n, W, _route_spec(4, 2, 1, 1, 1.5))
    assert ids.tolist() == [[3, 0]]                                # 0.27 + 1 beats 0.88: the correction chooses ...
    assert torch.allclose(wts, t64([[1.5 * float(s[3]), 1.5 * float(s[0])]]))      # ... and is not in the weight; no renormalising
    ids, _ = plain.route(n, {"router": router, "correction": torch.zeros(4, dtype=F64)}, _route_spec(4, 2, 1, 1, 1.5))
    assert ids.tolist() == [[0, 1]]


def test_router_keeps_groups_by_their_two_largest_and_bars_the_rest_even_with_negative_scores():
    # choice scores: group 0 = [0.9, 0.1, 0.1], group 1 = [0.6, 0.55, 0.0]: group 1 wins by its two largest (1.15 > 1.0),
    # though the single largest score lies in group 0
    logit = lambda p: math.log(p / (1 - p))
    n = t64([[1.0]])
    router = t64([[logit(0.9)], [logit(0.1)], [logit(0.1)], [logit(0.6)], [logit(0.55)], [logit(0.5)]])
    W = {"router": router, "correction": t64([0.0, 0.0, 0.0, 0.0, 0.0, -0.5])}
    ids, _ = plain.route(n, W, _route_spec(6, 2, 2, 1, 1.0))
    assert ids.tolist() == [[3, 4]]
    # three chosen: the third comes from the kept group although its choice score is 0 and every barred one is larger
    ids, _ = plain.route(n, W, _route_spec(6, 3, 2, 1, 1.0))
    assert ids.tolist() == [[3, 4, 5]]
    # all scores negative: the barred experts are out, not "zero and therefore best"
    W = {"router": router, "correction": t64([-2.0, -3.0, -3.0, -2.6, -2.6, -3.0])}
    ids, _ = plain.route(n, W, _route_spec(6, 2, 2, 1, 1.0))
    assert ids.tolist() == [[0, 1]]                                # group 0: -1.1 - 2.9 = -4.0 beats group 1: -2.0 - 2.05
    # a tie goes to the lower index
    W = {"router": t64([[0.3]] * 4), "correction": torch.zeros(4, dtype=F64)}
    assert plain.route(n, W, _route_spec(4, 2, 2, 1, 1.0))[0].tolist() == [[0, 1]]


def test_layer_scale_multiplies_each_sublayers_output_and_the_logits_pass_the_cap():
    raw = xu.ONLY["dense"]
    w = {k: v.double() for k, v in xu.make_weights(raw, 1).items()}
    toks = [4, 8, 15]
    seen = {}
    logits = plain.forward(raw, w, toks, on_layer=lambda i, x: seen.__setitem__(i, x.clone()))
    cap = raw["logit_softcap"]
    assert logits.abs().max() < cap
    h = plain.layer_norm(seen[0], w["final.norm"], raw["norm"]["eps"])
    assert torch.allclose(logits, cap * torch.tanh(h @ w["head"].T / cap))
    # the stream after the layer: embedding times its scale, plus ls1 * mixer, plus ls2 * feed-forward
    w0 = dict(w)
    w0["l0.ls1"] = torch.zeros_like(w["l0.ls1"])
    w0["l0.ls2"] = torch.zeros_like(w["l0.ls2"])
    plain.forward(raw, w0, toks, on_layer=lambda i, x: seen.__setitem__("bare", x.clone()))
    assert torch.allclose(seen["bare"], w["embed"][toks] * raw["embedding"]["scale"])
    w1 = dict(w0)
    w1["l0.ls2"] = w["l0.ls2"]
    plain.forward(raw, w1, toks, on_layer=lambda i, x: seen.__setitem__("ff", x.clone()))
    n = plain.layer_norm(seen["bare"], w["l0.norm2"], raw["norm"]["eps"])
    sub = {k[len("l0.mlp."):]: v for k, v in w.items() if k.startswith("l0.mlp.")}
    assert torch.allclose(seen["ff"], seen["bare"] + plain.dense_ff(n, sub) * w["l0.ls2"])


def test_configuration_reads_every_size_and_refuses_what_it_cannot_run():
    from tuff_amd.config.base import ConfigError
    from tuff_amd.models.registry import build_model, config_from_dict
    for name, raw in xu.CONFIGS.items():
        cfg = config_from_dict(raw)
        assert cfg.unknown_keys == [] and config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict(), name
        model = build_model(cfg)
        assert len(model.schedule) == len(raw["layers"]), name
    bad = [
        lambda r: r["layers"][0].update(type="conv"),
        lambda r: r["layers"][0]["mixer"].pop("state"),
        lambda r: r["layers"][0]["mixer"].update(groups=3),
        lambda r: r["layers"][0]["mixer"].update(norm_groups=5),
        lambda r: r["layers"][1]["mixer"].pop("scale"),
        lambda r: r["layers"][2]["mixer"].update(kv_heads=3),
        lambda r: r["layers"][3]["mixer"].update(kv_from=3),
        lambda r: r["layers"][3]["mixer"].update(kv_from=0),           # a layer without latent rows
        lambda r: r["layers"][3]["mixer"].update(kv_rank=24),          # not the rank of the rows it reads
        lambda r: r["layers"][1]["mlp"]["router"].update(top=9),
        lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(count=3),
        lambda r: r["layers"][1]["mlp"]["router"]["groups"].update(keep=1),          # four chosen of the two experts kept
        lambda r: r["layers"][1]["mlp"]["router"].update(scale="large"),
        lambda r: r["layers"][0]["mlp"].update(kind="gated"),
        lambda r: r["norm"].update(eps=0),
        lambda r: r.update(logit_softcap=-1.0),
        lambda r: r.pop("vocab"),
    ]
    # a router without groups or scale: one group of all experts, plain scores
    bare = copy.deepcopy(xu.X_MIXED)
    bare["layers"][3]["mlp"]["router"] = {"experts": 4, "top": 2}
    ffn = build_model(config_from_dict(bare)).blocks[3].ffn
    assert (ffn.route_groups, ffn.route_keep, ffn.route_scale) == (1, 1, 1.0)
    for i, spoil in enumerate(bad):
        raw = copy.deepcopy(xu.X_MIXED)
        spoil(raw)
        with pytest.raises(ConfigError):
            config_from_dict(raw)
            pytest.fail(f"case {i} was accepted")


def test_declared_tensors_and_caches():
    from tuff_amd.cache.manager import CacheLayout
    from tuff_amd.models.registry import build_model, config_from_dict
    from tuff_amd.parts.base import FixedState, PagedKV
    model = build_model(config_from_dict(xu.X_MIXED))
    decls = {d.name: tuple(d.shape) for d in model.weight_decls()}
    assert decls["l0.mix.in"] == (2 * 32 + 2 * 2 * 16 + 4, 64) and decls["l0.mix.conv"] == (32 + 64, 4) and decls["l0.mix.conv.b"] == (96,)
    assert decls["l0.mix.dt_bias"] == decls["l0.mix.A_log"] == decls["l0.mix.D"] == (4,) and decls["l0.mix.norm"] == (32,)
    assert decls["l0.mlp.gate"] == (40, 64) and decls["l0.ls1"] == decls["l0.ls2"] == (64,)
    assert decls["l1.mix.q"] == (32, 64) and decls["l1.mix.dkv"] == (32, 64) and decls["l1.mix.dkv.norm"] == (32,)
    assert decls["l1.mix.uk"] == (32, 32) and decls["l1.mix.uv"] == (48, 32) and decls["l1.mix.sink"] == (2,)
    assert decls["l1.mlp.e3.gate"] == (40, 64) and decls["l1.mlp.router"] == (4, 64) and decls["l1.mlp.correction"] == (4,)
    assert decls["l2.mix.q"] == (32, 64) and decls["l2.mix.v"] == (32, 64) and decls["l2.mix.q.conv"] == (32, 2)
    assert decls["l2.mix.a"] == decls["l2.mix.b"] == (4, 64) and decls["l2.mix.dt_bias"] == (4,) and decls["l2.mix.g"] == (32, 64)
    assert decls["l2.mix.norm"] == (8,) and "l2.norm2" not in decls and "l2.ls2" not in decls
    assert "l3.mix.dkv" not in decls and "l3.mix.dkv.norm" not in decls and decls["l3.mix.uk"] == (24, 32) and decls["l3.mix.sink"] == (3,)
    # one paged entry for the two latent layers (the reader runs on the writer's), a tail and a matrix state for each recurrence
    layout = CacheLayout.from_specs(model.cache_specs)
    assert list(layout.paged.values()) == [PagedKV(1, 32, None)]
    assert model.schedule[3].cache == model.schedule[1].cache and not model.schedule[3].writes
    states = sorted(layout.states.values(), key=lambda s: s.shape)
    assert FixedState((3, 96)) in states and FixedState((4, 16, 8)) in states          # mamba2: taps - 1 rows of x, B, C; [H, N, P]
    assert FixedState((1, 96)) in states and FixedState((4, 16, 8)) in states          # delta: q, k, v rows; [H, D, Dv]
    assert FixedState((2, 8, 24)) in states and len(states) == 6
    # one tap keeps no tail
    odd = build_model(config_from_dict(xu.X_ODD))
    assert sum(isinstance(s, FixedState) and len(s.shape) == 2 for s in odd.cache_specs.values()) == 1


def test_random_model_folder_round_trip(tmp_path):
    from tuff_amd.models.registry import build_model, config_from_dict, load_config
    from tuff_amd.weights.loader import Checkpoint
    from tuff_amd.weights.random_init import write_random_model
    cfg = config_from_dict(xu.X_MIXED)
    write_random_model(cfg, str(tmp_path), seed=3)
    assert load_config(str(tmp_path)).to_dict() == cfg.to_dict()
    assert set(Checkpoint(str(tmp_path)).names()) == {d.name for d in build_model(cfg).weight_decls()}
