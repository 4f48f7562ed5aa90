"""Loluzen on the GPU against the plain implementation (tests/plain/loluzen_plain.py): every mechanism
alone, whole prompts against token-by-token decoding, portions down to two tokens, batches of unequal
requests, pages and slots used again, far keys and page borders, first tokens, long decoding, sizes
nobody tuned the kernels for, and greedy generation through the scheduler and the command line."""
import functools
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import loluzen_util as lu
import util
from plain import loluzen_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
WHOLE = ["mixed", "wide", "odd", "plain"]


@functools.lru_cache(maxsize=None)
def model(name: str, seed: int = 0, peaky: float = 1.0):
    raw = lu.CONFIGS[name]
    w = lu.make_weights(raw, seed, peaky)
    folder = os.path.join(util._TMP.name, f"loluzen_{name}_{seed}_{peaky}")
    return lu.write_folder(raw, w, folder), raw, w


@functools.lru_cache(maxsize=512)
def _plain(name, seed, peaky, tokens, scale):
    _, raw, w = model(name, seed, peaky)
    if scale is None:
        return plain.forward(raw, w, list(tokens))
    return plain.forward(raw, w, list(tokens), rnd=lambda t: plain.bf16_round(t * scale) / scale)


def expected(name, tokens, seed=0, peaky=1.0) -> util.Expected:
    """Exact logits, and three realizations of the logits of a model that rounds its activations to bfloat16."""
    tokens = tuple(tokens)
    return util.Expected(_plain(name, seed, peaky, tokens, None),
                         [_plain(name, seed, peaky, tokens, s) for s in util.REALIZATION_SCALES])


def engine(name, dtype, seed=0, peaky=1.0, **kw):
    from tuff_amd.engine.engine import Engine
    folder, _, _ = model(name, seed, peaky)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Engine.from_folder(folder, dtype=dtype, poison_cache=True, **kw)


def requests(name, lengths, seed=0):
    V = lu.CONFIGS[name]["vocab"]
    return {f"r{i}": util.rand_tokens(n, V, seed * 100 + i) for i, n in enumerate(lengths)}


def compare(name, dtype, got, reqs, seed=0, peaky=1.0, what=""):
    """float32: every request against the exact logits.  bfloat16: the rows of all requests together against the
    rounding model's error (a request of one or two rows alone scatters too much for a bound on a mean)."""
    exp = {rid: expected(name, toks, seed, peaky) for rid, toks in reqs.items()}
    if dtype == "float32":
        for rid in reqs:
            util.assert_close_f32(got[rid], exp[rid], f"{what} {name} {rid}")
        return
    rids = list(reqs)
    for r in rids:
        assert torch.isfinite(got[r]).all(), f"{what} {name} {r}: non-finite logits"
    if sum(len(reqs[r]) for r in rids) < 8:
        return
    want = util.Expected(torch.cat([exp[r].want for r in rids]),
                         [torch.cat([exp[r].rounded[i] for r in rids]) for i in range(len(util.REALIZATION_SCALES))])
    util.assert_close_bf16(torch.cat([got[r] for r in rids]), want, f"{what} {name} bfloat16")


def check(name, dtype, plan, reqs, seed=0, peaky=1.0, **kw):
    eng = engine(name, dtype, seed, peaky, **kw)
    got = util.run_plan(eng, plan)
    eng.manager.check()
    assert not eng.manager.live()
    compare(name, dtype, got, reqs, seed, peaky)
    return eng, got


def all_single(reqs):
    return util.plan_tail(reqs, tail=10 ** 6)


# ------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", [n for n in lu.CONFIGS if n.startswith("only_")])
def test_each_mechanism_alone(gpu, name, dtype):
    reqs = requests(name, [37, 1, 9])
    check(name, dtype, util.plan_whole(reqs), reqs)
    check(name, dtype, util.plan_chunks(reqs, sizes=(2, 5, 1, 3, 16, 2)), reqs)


# -------------------------------------------------------------- whole models under every plan
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", WHOLE)
def test_whole_prompts(gpu, name, dtype):
    reqs = requests(name, [90, 1, 2, 33])
    check(name, dtype, util.plan_whole(reqs), reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", WHOLE)
def test_prompt_then_single_tokens_and_single_tokens_from_the_start(gpu, name, dtype):
    reqs = requests(name, [70, 40], seed=1)
    check(name, dtype, util.plan_tail(reqs, tail=32), reqs, seed=1)
    first = requests(name, [24], seed=2)        # the first tokens one by one: states start at zero, taps reach before the start
    check(name, dtype, all_single(first), first, seed=1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", WHOLE)
def test_portions_of_changing_size(gpu, name, dtype):
    reqs = requests(name, [150, 61], seed=3)
    check(name, dtype, util.plan_chunks(reqs), reqs)
    small = {"r1": reqs["r1"]}                  # portions shorter than the convolutions' taps
    check(name, dtype, util.plan_chunks(small, sizes=(2, 2, 3, 2, 1, 2)), small)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", WHOLE)
def test_batches_of_unequal_requests_with_pages_and_slots_used_again(gpu, name, dtype):
    reqs = requests(name, [5, 77, 130, 2, 40, 64, 19, 95, 33], seed=4)
    plan = util.plan_mixed(reqs, seed=4, max_live=3)
    peak = util.live_tokens_peak(plan)
    eng, got = check(name, dtype, plan, reqs, max_tokens=peak, max_requests=3)
    assert eng.manager.groups[0].pool.allocations > eng.manager.groups[0].pool.num_pages       # pages came back and went out again
    # once more on the same engine: every page and slot has been used before, and holds NaN or another request's state
    again = util.run_plan(eng, plan)
    if dtype == "float32":
        for rid in reqs:
            assert torch.equal(again[rid], got[rid]), rid
    else:
        compare(name, dtype, again, reqs, what="second run")


@pytest.mark.parametrize("name", ["mixed", "wide", "odd"])
def test_float32_logits_do_not_depend_on_the_plan(gpu, name):
    """The same bits whether a prompt comes whole, in portions, token by token or beside other requests, with
    recorded steps or without."""
    reqs = requests(name, [83, 30, 47], seed=5)
    plans = [util.plan_whole(reqs), util.plan_chunks(reqs), all_single(reqs), util.plan_mixed(reqs, seed=1)]
    base = util.run_plan(engine(name, "float32"), plans[0])
    for i, plan in enumerate(plans[1:]):
        for graphs in (True, False):
            got = util.run_plan(engine(name, "float32", use_graphs=graphs), plan)
            for rid in reqs:
                assert torch.equal(got[rid], base[rid]), f"plan {i + 1}, graphs {graphs}, {rid}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(gpu, dtype):
    reqs = requests("mixed", [330], seed=6)
    check("mixed", dtype, util.plan_tail(reqs, tail=325), reqs)


# --------------------------------------------------------------- far keys and page borders
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["only_attention", "only_attention_equal", "only_attention_bare", "only_pair", "only_pair_wide"])
def test_peaky_attention_far_keys_in_prompts_and_in_decoding(gpu, name, dtype):
    """W_q and W_k scaled up: a few keys hold the weight, anywhere in hundreds; a key lost, taken twice or read
    from a neighbour's page moves the logits."""
    reqs = requests(name, [420, 300], seed=8)
    check(name, dtype, util.plan_tail(reqs, tail=70), reqs, peaky=4.0)
    check(name, dtype, util.plan_chunks(reqs, sizes=(15, 1, 16, 17, 2, 31, 33, 64, 63, 65)), reqs, peaky=4.0)


def _mixed_heads(q, k, v, r1, r2, talk, scale):
    """The last query of q [n, H, dk] over k [n, G, dk], v [n, G, dv], float64 -> [H, dv]: a logarithmic distance penalty
    off the scaled scores, softmax, the heads' weights mixed by talk, each head on its own kv head's values."""
    n, H, G = q.shape[0], q.shape[1], k.shape[1]
    dist = torch.arange(n - 1, -1, -1, dtype=torch.float64)
    p = torch.stack([torch.softmax((k[:, h // (H // G)] @ q[-1, h]) * scale - r1[h] * torch.log1p(r2[h] * dist), 0) for h in range(H)])
    mixed = talk @ p
    return torch.stack([mixed[h] @ v[:, h // (H // G)] for h in range(H)])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dk, dv, H, G", [(16, 16, 4, 2), (64, 64, 8, 2), (24, 40, 3, 1), (128, 128, 2, 2), (80, 48, 4, 4),
                                          (64, 128, 6, 3), (256, 256, 2, 1), (32, 32, 12, 1), (40, 8, 1, 1)])
def test_attention_with_mixed_heads_one_key_stands_out(gpu, dk, dv, H, G, dtype):
    """The pair's attention mixer alone, its projections identities: one key, at the start, far back, at a page's border
    or the last, lines up with the last query so that it holds most of the weight against the distance penalty; the
    mixing matrix has negative and large entries.  The step's queries see it from a prompt's portion and from single
    tokens.  Pages are scattered and everything else in the pool is NaN."""
    from tuff_amd.cache.manager import CacheLayout, CacheManager
    from tuff_amd.cache.storage import CacheStorage
    from tuff_amd.engine.batch import StepEntry, build_context
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import Runtime
    ps = 16
    gen = torch.Generator().manual_seed(dk + dv + H)
    width = H * dk + G * dk + G * dv
    names = {k: k for k in ("q", "k", "v", "o", "q.b", "k.b", "v.b", "r1", "r2", "talk")}
    mixer = AttentionMixer(width, H, G, dk, value_dim=dv, scale=0.4, names=names)
    eye = torch.eye(width)
    r1, r2 = 0.2 + torch.rand(H, generator=gen), 0.1 + 2.0 * torch.rand(H, generator=gen)
    talk = torch.randn(H, H, generator=gen)
    weights = {"q": eye[:H * dk], "k": eye[H * dk:H * dk + G * dk], "v": eye[H * dk + G * dk:], "o": torch.eye(H * dv),
               "q.b": torch.zeros(H * dk), "k.b": torch.zeros(G * dk), "v.b": torch.zeros(G * dv), "r1": r1, "r2": r2, "talk": talk}
    weights = {n: t.to(dtype).to(gpu) for n, t in weights.items()}
    mixer.bind(weights, Runtime(gpu, dtype))
    r1, r2, talk = (weights[n].double().cpu() for n in ("r1", "r2", "talk"))
    layout = CacheLayout.from_specs({0: mixer.cache_spec()})
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for n, special in [(1, 0), (17, 0), (257, 15), (257, 16), (300, 255), (300, 256), (700, 3), (129, 128), (200, 136)]:
        mgr = CacheManager(layout, ps, 64, 2)
        store = CacheStorage(mgr, dtype, gpu, poison=True)
        mgr.admit("pad")
        mgr.extend("pad", 40)                               # the request's pages do not start at page 0
        mgr.admit("a")
        x = torch.randn(n, width, generator=gen) * 0.5
        qrows = x[:, :H * dk].view(n, H, dk)
        krows = x[:, H * dk:H * dk + G * dk].view(n, G, dk)
        for g in range(G):                                   # the special key lines up with the last query's heads
            krows[special, g] = qrows[n - 1, g * (H // G)] * (6.0 + 1.5 * math.log1p(n))
        x = x.to(dtype)
        xf = x.double()
        qf = xf[:, :H * dk].view(n, H, dk)
        kf = xf[:, H * dk:H * dk + G * dk].view(n, G, dk)
        vf = xf[:, H * dk + G * dk:].view(n, G, dv)
        tail = min(3, n - 1)
        steps = [list(range(0, n - tail))] + [[i] for i in range(n - tail, n)] if n > tail else [[0]]
        for rows in steps:
            if not rows:
                continue
            mgr.extend("a", len(rows))
            ctx = build_context([StepEntry("a", [0] * len(rows), [])], mgr, gpu, 10)
            res = torch.zeros(len(rows), H * dv, dtype=torch.float32, device=gpu)
            mixer.forward(x[rows].to(gpu).contiguous(), ctx, store.views[0], res)
            for at in {len(rows) - 1, len(rows) // 2}:       # the last query of the step, and one in a portion's middle
                i = rows[at]
                want = _mixed_heads(qf[:i + 1], kf[:i + 1], vf[:i + 1], r1, r2, talk, 0.4).reshape(-1)
                err = (res[at].double().cpu() - want).abs().max()
                assert err <= tol * max(1.0, float(want.abs().max())), (n, special, i, float(err))


def _paged_case(gpu, H, Hkv, hd, vd, reqs, opts, ps=16, seed=0):
    """Scattered pages of random bfloat16 keys and values for requests (tokens before the step, tokens of the step), queries,
    and the options' tensors; everything a kernel's launch takes."""
    gen = torch.Generator().manual_seed(seed)
    rnd = lambda *shape: torch.randn(*shape, generator=gen)
    R, T = len(reqs), sum(n for _, n in reqs)
    longest = max(c + n for c, n in reqs)
    nblk = -(-longest // ps)
    P = R * nblk + 3
    table = torch.randperm(P, generator=gen)[:R * nblk].view(R, nblk).int().to(gpu)
    i32 = lambda a: torch.tensor(a, dtype=torch.int32, device=gpu)
    req_of, pos, info, t = [], [], [], 0
    for r, (c, n) in enumerate(reqs):
        info.append((t, n, c, 0)); req_of += [r] * n; pos += list(range(c, c + n)); t += n
    window, sinks, slopes, logd, talk, gate = opts
    case = dict(q=(rnd(T, H * hd) * 1.5).bfloat16().to(gpu), k=rnd(P, Hkv, ps, hd).bfloat16().to(gpu), v=rnd(P, Hkv, vd, ps).bfloat16().to(gpu),
                table=table, req_of=i32(req_of), pos=i32(pos), info=i32(info), longest=longest, T=T, window=window,
                sinks=(rnd(H) + 1).to(gpu) if sinks else None, slopes=(torch.rand(H, generator=gen) * 0.1).to(gpu) if slopes else None,
                logd=((torch.rand(H, generator=gen) + 0.2).to(gpu), (torch.rand(H, generator=gen) * 2 + 0.1).to(gpu)) if logd else None,
                talk=rnd(H, H).to(gpu) if talk else None, gates=rnd(T, H).to(gpu) if gate else None)
    return case


def _general(c, H, Hkv, hd, vd, ps=16):
    """The one-wave-a-head kernel (float32 weights; held to the plain functions by the float32 tests above), then the
    heads' mixing and gates: [T, H * vd] float32."""
    from tuff_amd.csrc import ops
    mixed = c["talk"] is not None
    o = torch.zeros((c["T"], H * Hkv * vd) if mixed else (c["T"], H * vd), dtype=torch.float32 if mixed else torch.bfloat16, device=c["q"].device)
    ops.attention_general(c["q"], c["k"], c["v"], o, block_table=c["table"], req_of_token=c["req_of"], positions=c["pos"], H=H, Hkv=Hkv,
                          hd=hd, page_size=ps, window=c["window"], scale=0.2, vd=vd, sinks=c["sinks"], slopes=c["slopes"],
                          log_distance=c["logd"], all_values=mixed)
    if not mixed and c["gates"] is None:
        return o.float()
    out = torch.zeros(c["T"], H * vd, dtype=o.dtype, device=o.device)
    ops.head_mix_gate(o, out, H=H, Hkv=Hkv, vd=vd, talk=c["talk"], gates=c["gates"])
    return out.float()


SHAPES = [(4, 2, 64, 64), (4, 4, 80, 48), (6, 3, 24, 40), (2, 1, 128, 128), (8, 2, 40, 16), (2, 2, 256, 64), (40, 2, 16, 8), (3, 3, 8, 256)]
# (window, sinks, slopes, logarithmic penalty, mixed heads, gates)
OPTIONS = [(0, 0, 0, 0, 0, 0), (48, 0, 0, 0, 0, 0), (0, 1, 0, 0, 0, 1), (300, 1, 0, 0, 0, 0), (0, 0, 1, 0, 0, 0), (0, 0, 0, 1, 0, 0),
           (0, 0, 0, 1, 1, 1), (100, 1, 0, 1, 1, 0)]


@pytest.mark.parametrize("H, Hkv, hd, vd", SHAPES)
def test_prompt_kernel_in_its_wide_form_against_the_general_kernel(gpu, H, Hkv, hd, vd):
    """Portions at the start, far into a request and across page and step borders, a single token among them; float32
    sums where the heads are mixed agree to float32's rounding: the weights keep their precision through the matrix cores."""
    from tuff_amd.csrc import ops
    reqs = [(0, 70), (130, 5), (300, 1), (17, 200)]
    for opts in OPTIONS:
        c = _paged_case(gpu, H, Hkv, hd, vd, reqs, opts, seed=H + hd)
        c["gates"] = None
        want = _general(c, H, Hkv, hd, vd)
        mixed = c["talk"] is not None
        o = torch.zeros((c["T"], H * Hkv * vd) if mixed else (c["T"], H * vd), dtype=torch.float32 if mixed else torch.bfloat16, device=gpu)
        blocks = torch.from_numpy(ops.query_blocks(np.array([n for _, n in reqs]), H // Hkv, 8, np.array([a + n for a, n in reqs]))).to(gpu)
        ops.attention_prefill_wide(c["q"], c["k"], c["v"], o, block_table=c["table"], blocks=blocks, req_info=c["info"], H=H, Hkv=Hkv, hd=hd,
                                   vd=vd, page_size=16, max_ctx_len=c["longest"], window=c["window"], scale=0.2, sinks=c["sinks"],
                                   slopes=c["slopes"], log_distance=c["logd"], all_values=mixed)
        if mixed:
            got = torch.zeros(c["T"], H * vd, dtype=torch.float32, device=gpu)
            ops.head_mix_gate(o, got, H=H, Hkv=Hkv, vd=vd, talk=c["talk"], gates=None)
        else:
            got = o.float()
        tol = 3e-5 if mixed else 0.01
        assert (got - want).abs().max() <= tol * max(1.0, float(want.abs().max())), opts


@pytest.mark.parametrize("H, Hkv, hd, vd", SHAPES)
def test_single_token_kernels_with_float32_weights_against_the_general_kernel(gpu, H, Hkv, hd, vd):
    """Single tokens at the first position, on both sides of a part's 256 keys and far behind them."""
    from tuff_amd.csrc import ops
    reqs = [(n, 1) for n in (0, 5, 255, 256, 257, 700, 1023, 15)]
    for opts in OPTIONS:
        c = _paged_case(gpu, H, Hkv, hd, vd, reqs, opts, seed=H + vd)
        want = _general(c, H, Hkv, hd, vd)
        got = torch.zeros(c["T"], H * vd, dtype=torch.float32, device=gpu)
        ops.attention_decode_exact(c["q"], c["k"], c["v"], got, block_table=c["table"], req_of_token=c["req_of"], positions=c["pos"], H=H,
                                   Hkv=Hkv, hd=hd, vd=vd, page_size=16, max_ctx_len=c["longest"], window=c["window"], scale=0.2,
                                   sinks=c["sinks"], slopes=c["slopes"], log_distance=c["logd"], talk=c["talk"], gates=c["gates"])
        tol = 3e-5 if c["talk"] is not None else 0.01            # (the general kernel's own output is bfloat16 where heads are not mixed)
        assert (got - want).abs().max() <= tol * max(1.0, float(want.abs().max())), opts


def test_forget_scan_carries_its_state_across_any_cut(gpu):
    """The recurrence's kernel on its own, at key sizes on both sides of a wave's 64 lanes and value sizes of one and
    several blocks: a sequence in one call against the same sequence in portions of 1, 2 and more through the state, in
    a slot between slots of NaN, against the plain loop.  Gates near 0 and near 1 are among them."""
    from tuff_amd.csrc import ops
    gen = torch.Generator().manual_seed(5)
    for H, D, Dv in [(2, 16, 16), (3, 40, 72), (1, 100, 130), (2, 200, 24), (1, 256, 8), (4, 48, 64), (1, 1, 1)]:
        n = 23
        x = torch.randn(n, 2 * H * D + H * Dv, generator=gen)
        x[:, H * D:2 * H * D] *= 6.0                                  # gate logits: many gates at their bounds
        fb, lower = torch.randn(H * D, generator=gen), 0.02 + 0.96 * torch.rand(H * D, generator=gen)
        xd = x.double()
        q = torch.nn.functional.silu(xd[:, :H * D]).view(n, H, D)
        f = (lower.double() + (1 - lower.double()) * torch.sigmoid(xd[:, H * D:2 * H * D] + fb.double())).view(n, H, D)
        v = xd[:, 2 * H * D:].view(n, H, Dv)
        S = torch.zeros(H, D, Dv, dtype=torch.float64)
        want = torch.zeros(n, H, Dv, dtype=torch.float64)
        for t in range(n):
            S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
            want[t] = torch.einsum("hij,hi->hj", S, q[t])
        dev = lambda t: t.to(gpu).contiguous()
        i32 = lambda *v_: torch.tensor(v_, dtype=torch.int32, device=gpu)
        for cuts in ([n], [1] * n, [2, 1, 7, 2, 11]):
            state = torch.full((3, H, D, Dv), float("nan"), device=gpu)
            state[1] = 0
            out, pos = [], 0
            for c in cuts:
                o = torch.empty(c, H * Dv, device=gpu)
                ops.forget_scan(dev(x[pos:pos + c]), dev(fb), dev(lower), state, o, q_start=i32(0), q_len=i32(c),
                                state_slot=i32(1), H=H, D=D, Dv=Dv)
                out.append(o.cpu())
                pos += c
            got = torch.cat(out).view(n, H, Dv).double()
            assert (got - want).abs().max() <= 2e-5 * max(1.0, float(want.abs().max())), (H, D, Dv, cuts)
            assert (state[1].double().cpu() - S).abs().max() <= 2e-5 * max(1.0, float(S.abs().max())), (H, D, Dv, cuts)
            assert torch.isnan(state[0]).all() and torch.isnan(state[2]).all()


# ------------------------------------------------------------------- generation, command line
def test_greedy_generation_through_the_scheduler(gpu):
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    reqs = requests("mixed", [5, 21, 1, 12, 30, 8], seed=9)
    _, raw, w = model("mixed")
    eng = engine("mixed", "float32", max_tokens=512, max_requests=3)
    llm = LLM(engine=eng, max_num_seqs=3, max_batched_tokens=16, ctx_size=128, ignore_eos=True)
    outs = llm.generate(list(reqs.values()), SamplingParams(temp=0.0, max_new_tokens=10, ignore_eos=True))
    for g, prompt in zip(outs, reqs.values()):
        assert list(g.token_ids) == plain.greedy(raw, w, prompt, 10), prompt
    eng.manager.check()
    assert not eng.manager.live()


def test_command_line_and_trace_replay(gpu, tmp_path):
    folder, raw, w = model("wide")
    prompt = util.rand_tokens(9, raw["vocab"], 3)
    p = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--prompt-ids",
                        ",".join(map(str, prompt)), "--dump-tokens", "-n", "6", "--dtype", "fp32", "--temp", "0"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(x) for x in p.stdout.split()] == plain.greedy(raw, w, prompt, 6)
    q = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--inspect"],
                       capture_output=True, text=True, timeout=300)
    assert q.returncode == 0 and "PairMixer" in q.stdout and "ForgetGateMixer" in q.stdout, q.stderr[-2000:]
    # the trace runner: a mixed plan through a child process, four slots, a pool no larger than the plan's peak
    reqs = requests("wide", [50, 3, 70, 20, 31], seed=10)
    plan = util.plan_mixed(reqs, seed=2)
    out = tmp_path / "out"
    cmd = [sys.executable, os.path.join(util.ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
           "--out", str(out), "--max-tokens", str(util.live_tokens_peak(plan))]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in plan:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {s['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    fed = {rid: 0 for rid in reqs}
    for s in plan:
        n_want = sum(len(e["want"]) for e in s["entries"])
        data = torch.from_numpy(np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(n_want, raw["vocab"]).copy())
        i = 0
        for e in s["entries"]:
            want = expected("wide", reqs[e["id"]]).want
            rows = [fed[e["id"]] + w_ for w_ in e["want"]]
            util.assert_close_f32(data[i:i + len(rows)], want[rows], f"step {s['step']} {e['id']}")
            i += len(rows)
            fed[e["id"]] += len(e["tokens"])
