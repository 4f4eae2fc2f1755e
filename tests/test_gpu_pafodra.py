"""Pafodra on the GPU against the plain implementation (tests/plain/pafodra_plain.py): every mechanism
alone, whole prompts against token-by-token decoding, portions down to two tokens, batches of unequal
requests, pages and slots used again, far keys and page borders, first tokens, long decoding, sizes
nobody tuned the kernels for, and greedy generation through the scheduler and the command line."""
import functools
import math
import os
import subprocess
import sys

import pytest
import torch

import pafodra_util as pu
import util
from plain import pafodra_plain as plain

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]


@functools.lru_cache(maxsize=None)
def model(name: str, seed: int = 0, loud_attention: float = 1.0):
    raw = pu.CONFIGS[name]
    w = pu.make_weights(raw, seed, loud_attention)
    folder = os.path.join(util._TMP.name, f"pafodra_{name}_{seed}_{loud_attention}")
    return pu.write_folder(raw, w, folder), raw, w


@functools.lru_cache(maxsize=512)
def _plain(name, seed, loud, tokens, scale):
    _, raw, w = model(name, seed, loud)
    if scale is None:
        return plain.forward(raw, w, list(tokens))
    return plain.forward(raw, w, list(tokens), rnd=lambda t: plain.bf16_round(t * scale) / scale)


CLOSE_CALL = 0.05       # of the router logits' spread: below it, bfloat16 rounding may choose another expert


@functools.lru_cache(maxsize=512)
def rows_before_a_close_call(name, seed, loud, tokens) -> int:
    """How many leading tokens of the sequence have no router decision that rounding could turn (a token's
    logits depend on the tokens before it only)."""
    _, raw, w = model(name, seed, loud)
    margins = []
    plain.forward(raw, w, list(tokens), margins_out=margins)
    n = len(tokens)
    for m in margins:
        close = torch.nonzero(m < CLOSE_CALL)
        if len(close):
            n = min(n, int(close[0]))
    return n


def expected(name, tokens, seed=0, loud=1.0) -> util.Expected:
    """Exact logits, and three realizations of the logits of a model that rounds its activations to bfloat16."""
    tokens = tuple(tokens)
    return util.Expected(_plain(name, seed, loud, tokens, None),
                         [_plain(name, seed, loud, tokens, s) for s in util.REALIZATION_SCALES])


def engine(name, dtype, seed=0, loud=1.0, **kw):
    from tuff_amd.engine.engine import Engine
    folder, _, _ = model(name, seed, loud)
    kw.setdefault("page_size", 16)
    kw.setdefault("max_tokens", 1024)
    kw.setdefault("max_requests", 4)
    return Engine.from_folder(folder, dtype=dtype, poison_cache=True, **kw)


def requests(name, lengths, seed=0):
    V = pu.CONFIGS[name]["vocab"]
    return {f"r{i}": util.rand_tokens(n, V, seed * 100 + i) for i, n in enumerate(lengths)}


def check(name, dtype, plan, reqs, seed=0, loud=1.0, **kw):
    eng = engine(name, dtype, seed, loud, **kw)
    got = util.run_plan(eng, plan)
    eng.manager.check()
    assert not eng.manager.live()
    compare(name, dtype, got, reqs, seed, loud)
    return eng, got


def compare(name, dtype, got, reqs, seed=0, loud=1.0, what=""):
    """float32: every request against the exact logits.  bfloat16: the rows of all requests together against the
    rounding model's error (a request of one or two rows alone scatters too much for a bound on a mean)."""
    exp = {rid: expected(name, toks, seed, loud) for rid, toks in reqs.items()}
    if dtype == "float32":
        for rid in reqs:
            util.assert_close_f32(got[rid], exp[rid], f"{what} {name} {rid}")
        return
    # A router's choice that hangs on less than rounding moves is no test of arithmetic: a request counts up to
    # its first such token (float32 covers the rest).
    rids = list(reqs)
    keep = {r: rows_before_a_close_call(name, seed, loud, tuple(reqs[r])) for r in rids}
    for r in rids:
        assert torch.isfinite(got[r]).all(), f"{what} {name} {r}: non-finite logits"
    if sum(keep.values()) < 8:
        return
    want = util.Expected(torch.cat([exp[r].want[:keep[r]] for r in rids]),
                         [torch.cat([exp[r].rounded[i][:keep[r]] for r in rids]) for i in range(len(util.REALIZATION_SCALES))])
    util.assert_close_bf16(torch.cat([got[r][:keep[r]] for r in rids]), want, f"{what} {name} bfloat16")


def all_single(reqs):
    return util.plan_tail(reqs, tail=10 ** 6)


# ------------------------------------------------------------------------ mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", [n for n in pu.CONFIGS if n.startswith("only_")])
def test_each_mechanism_alone(gpu, name, dtype):
    reqs = requests(name, [37, 1, 9])
    check(name, dtype, util.plan_whole(reqs), reqs)
    check(name, dtype, util.plan_chunks(reqs, sizes=(2, 5, 1, 3, 16, 2)), reqs)


# -------------------------------------------------------------- whole models under every plan
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "wide", "odd"])
def test_whole_prompts(gpu, name, dtype):
    reqs = requests(name, [90, 1, 2, 33])
    check(name, dtype, util.plan_whole(reqs), reqs)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "wide", "odd"])
def test_prompt_then_single_tokens_and_single_tokens_from_the_start(gpu, name, dtype):
    reqs = requests(name, [70, 40], seed=1)
    check(name, dtype, util.plan_tail(reqs, tail=32), reqs, seed=1)
    first = requests(name, [24], seed=2)                 # the first tokens of a sequence, one by one: states start at zero
    check(name, dtype, all_single(first), first, seed=1)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "wide", "odd"])
def test_portions_of_changing_size(gpu, name, dtype):
    reqs = requests(name, [150, 61], seed=3)
    check(name, dtype, util.plan_chunks(reqs), reqs)
    small = {"r1": reqs["r1"]}
    check(name, dtype, util.plan_chunks(small, sizes=(2, 2, 3, 2, 1, 2)), small)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "wide", "odd"])
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


def test_steps_of_portions_recorded_in_sections(gpu):
    """The same step sizes again and again, so that steps with portions are recorded and replayed."""
    from tuff_amd.engine.engine import Engine
    reqs = requests("mixed", [96, 96, 96, 96], seed=7)
    plan = util.plan_chunks(reqs, sizes=(8,))
    eng, _ = check("mixed", "float32", plan, reqs)
    assert eng.section_replays > 0


# --------------------------------------------------------------- far keys and page borders
@pytest.mark.parametrize("dtype", DTYPES)
def test_peaky_attention_far_keys_in_prompts_and_in_decoding(gpu, dtype):
    """W_q and W_k scaled up: a few keys hold the weight, anywhere in hundreds; a key lost, taken twice or read
    from a neighbour's page moves the logits."""
    reqs = requests("only_attention", [420, 300], seed=8)
    for name in ("only_attention", "only_attention_equal"):
        check(name, dtype, util.plan_tail(reqs, tail=70), reqs, loud=4.0)
        check(name, dtype, util.plan_chunks(reqs, sizes=(15, 1, 16, 17, 2, 31, 33, 64, 63, 65)), reqs, loud=4.0)


def _sink_softmax(q, k, v, sink, scale):
    """q [H, dk], k [n, G, dk], v [n, G, dv] float64 -> [H, dv]"""
    H, G = q.shape[0], k.shape[1]
    out = []
    for h in range(H):
        g = h // (H // G)
        s = (k[:, g] @ q[h]) * scale
        top = max(float(s.max()), float(sink[h]))
        e = torch.exp(s - top)
        out.append((e[:, None] * v[:, g]).sum(0) / (e.sum() + math.exp(float(sink[h]) - top)))
    return torch.stack(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("dk, dv, H, G", [(16, 16, 4, 2), (64, 64, 8, 2), (24, 40, 3, 1), (128, 128, 2, 2), (256, 256, 2, 1),
                                          (32, 32, 24, 1)])
def test_attention_kernels_one_key_stands_out(gpu, dk, dv, H, G, dtype):
    """One key, at the start, far back, at a page's border or the last, is made to hold most of the weight
    beside a sink that holds a known share; the step's queries see it from a prompt's portion and from single
    tokens.  Pages are scattered and everything else in the pool is NaN."""
    from tuff_amd.parts.attention import AttentionMixer
    from tuff_amd.parts.base import Runtime
    from tuff_amd.engine.batch import StepEntry, build_context
    from tuff_amd.cache.manager import CacheLayout, CacheManager
    from tuff_amd.cache.storage import CacheStorage
    ps, d = 16, 32
    gen = torch.Generator().manual_seed(dk + dv)
    mixer = AttentionMixer(d, H, G, dk, value_dim=dv, scale=0.4, names={k: k for k in ("q", "k", "v", "o", "sink")})
    # identity-like projections: the mixer's input rows are q | k | v themselves
    width = H * dk + G * dk + G * dv
    mixer.d = width
    from tuff_amd.parts.linear import Linear
    mixer.qkv = Linear(["q", "k", "v"], width, [H * dk, G * dk, G * dv])
    mixer.out = Linear("o", H * dv, H * dv)
    eye = torch.eye(width)
    sink = torch.randn(H, generator=gen) + 2.0
    weights = {"q": eye[:H * dk], "k": eye[H * dk:H * dk + G * dk], "v": eye[H * dk + G * dk:], "o": torch.eye(H * dv), "sink": sink}
    weights = {n: t.to(dtype).to(gpu) for n, t in weights.items()}
    mixer.bind(weights, Runtime(gpu, dtype))
    layout = CacheLayout.from_specs({0: mixer.cache_spec()})
    for n, special in [(1, 0), (17, 0), (257, 15), (257, 16), (300, 255), (300, 256), (700, 3), (129, 128)]:
        mgr = CacheManager(layout, ps, 64, 2)
        store = CacheStorage(mgr, dtype, gpu, poison=True)
        mgr.admit("pad")
        mgr.extend("pad", 40)                               # the request's pages do not start at page 0
        mgr.admit("a")
        x = torch.randn(n, width, generator=gen) * 0.5
        qrows = x[:, :H * dk].view(n, H, dk)
        krows = x[:, H * dk:H * dk + G * dk].view(n, G, dk)
        krows[special] = 0
        for g in range(G):                                   # the special key lines up with the last query's heads
            krows[special, g] = qrows[n - 1, g * (H // G)] * 6.0
        x = x.to(dtype)
        xf = x.double()
        qf = xf[:, :H * dk].view(n, H, dk)
        kf = xf[:, H * dk:H * dk + G * dk].view(n, G, dk)
        vf = xf[:, H * dk + G * dk:].view(n, G, dv)
        want_last = _sink_softmax(qf[n - 1], kf, vf, sink.to(dtype).double(), 0.4).reshape(-1)
        tail = min(3, n - 1)
        steps = [list(range(0, n - tail))] + [[i] for i in range(n - tail, n)] if n > tail else [[0]]
        got = None
        for rows in steps:
            if not rows:
                continue
            mgr.extend("a", len(rows))
            ctx = build_context([StepEntry("a", [0] * len(rows), [])], mgr, gpu, 10)
            res = torch.zeros(len(rows), H * dv, dtype=torch.float32, device=gpu)
            mixer.forward(x[rows].to(gpu).contiguous(), ctx, store.views[0], res)
            got = res[-1].double().cpu()
            if len(rows) > 1:                                # a portion: check one query in its middle too
                i = rows[len(rows) // 2]
                mid = _sink_softmax(qf[i], kf[:i + 1], vf[:i + 1], sink.to(dtype).double(), 0.4).reshape(-1)
                tol = 1e-5 if dtype == torch.float32 else 2e-2
                assert (res[len(rows) // 2].double().cpu() - mid).abs().max() <= tol * max(1.0, float(mid.abs().max())), (n, special, "middle")
        tol = 1e-5 if dtype == torch.float32 else 2e-2
        assert (got - want_last).abs().max() <= tol * max(1.0, float(want_last.abs().max())), (n, special)


# ----------------------------------------------------------------------- kernels alone
def test_delta_scan_carries_its_state_across_any_cut(gpu):
    """The delta rule's kernel on its own, at head sizes with one, two and three blocks of value channels: a
    sequence in one call against the same sequence in portions of 1, 2 and more through the state, in a slot
    between slots of NaN, float32, against the plain loop."""
    from tuff_amd.csrc import ops
    gen = torch.Generator().manual_seed(5)
    for H, Hk, D, Dv in [(2, 2, 16, 16), (3, 1, 40, 72), (1, 1, 100, 130), (2, 1, 200, 24), (1, 1, 256, 8)]:
        n = 23
        rnd = lambda *s: torch.randn(*s, generator=gen)
        q, k, v = rnd(n, Hk * D), rnd(n, Hk * D), rnd(n, H * Dv)
        a, b, dtb, alog = rnd(n, H * D), rnd(n, H), rnd(H * D), rnd(H) * 0.5
        # plain: the delta rule's loop
        qn = q.view(n, Hk, D).double(); kn = k.view(n, Hk, D).double()
        qn = qn / torch.sqrt((qn * qn).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
        kn = kn / torch.sqrt((kn * kn).sum(-1, keepdim=True) + 1e-6)
        g = torch.exp(-torch.exp(alog.double())[None, :, None] * plain.softplus((a + dtb).double()).view(n, H, D))
        S = torch.zeros(H, D, Dv, dtype=torch.float64)
        want = torch.zeros(n, H, Dv, dtype=torch.float64)
        for t in range(n):
            kt, qt = kn[t].repeat_interleave(H // Hk, 0), qn[t].repeat_interleave(H // Hk, 0)
            S = g[t][:, :, None] * S
            e = torch.sigmoid(b[t].double())[:, None] * (v[t].view(H, Dv).double() - torch.einsum("hij,hi->hj", S, kt))
            S = S + kt[:, :, None] * e[:, None, :]
            want[t] = torch.einsum("hij,hi->hj", S, qt)
        dev = lambda t: t.to(gpu).contiguous()
        for cuts in ([n], [1] * n, [2, 1, 7, 2, 11]):
            state = torch.full((3, H, D, Dv), float("nan"), device=gpu)
            state[2] = 0
            out = []
            pos = 0
            for c in cuts:
                sl = slice(pos, pos + c)
                o = torch.empty(c, H * Dv, device=gpu)
                i32 = lambda *v_: torch.tensor(v_, dtype=torch.int32, device=gpu)
                ops.delta_scan(dev(q[sl]), dev(k[sl]), dev(v[sl]), dev(a[sl]), dev(dtb), dev(alog), dev(b[sl]), state, o,
                               q_start=i32(0), q_len=i32(c), state_slot=i32(2), H=H, Hk=Hk, D=D, Dv=Dv)
                out.append(o.cpu())
                pos += c
            got = torch.cat(out).view(n, H, Dv).double()
            assert (got - want).abs().max() <= 2e-5 * max(1.0, float(want.abs().max())), (H, Hk, D, Dv, cuts)


def test_moe_routing_ties_and_order(gpu):
    from tuff_amd.csrc import ops
    z = torch.tensor([[0.5, 2.0, 2.0, -1.0, 0.5], [3.0, -3.0, 0.0, 0.0, 9.0]], device=gpu)
    ids = torch.empty(2, 3, dtype=torch.int32, device=gpu)
    wts = torch.empty(2, 3, device=gpu)
    ops.moe_route(z, ids, wts, E=5, top=3)
    assert ids.cpu().tolist() == [[1, 2, 0], [4, 0, 2]]                     # the lower index wins a tie
    assert torch.allclose(wts.cpu(), torch.sigmoid(torch.tensor([[2.0, 2.0, 0.5], [9.0, 3.0, 0.0]])))
    ids1, wts1 = torch.empty(2, 1, dtype=torch.int32, device=gpu), torch.empty(2, 1, device=gpu)
    ops.moe_route(z, ids1, wts1, E=4, top=1)                                # a wider row than experts: the rest is not routed
    assert ids1.cpu().tolist() == [[1], [0]]


# ------------------------------------------------------------------- generation, command line
def _plain_greedy(name, prompt, n_new, seed=0):
    _, raw, w = model(name, seed)
    toks = list(prompt)
    for _ in range(n_new):
        toks.append(int(plain.forward(raw, w, toks)[-1].argmax()))
    return toks[len(prompt):]


def test_greedy_generation_through_the_scheduler(gpu):
    from tuff_amd.engine.llm import LLM
    from tuff_amd.sampling.params import SamplingParams
    reqs = requests("mixed", [5, 21, 1, 12, 30, 8], seed=9)
    eng = engine("mixed", "float32", max_tokens=512, max_requests=3)
    llm = LLM(engine=eng, max_num_seqs=3, max_batched_tokens=16, ctx_size=128, ignore_eos=True)
    outs = llm.generate(list(reqs.values()), SamplingParams(temp=0.0, max_new_tokens=10, ignore_eos=True))
    for g, prompt in zip(outs, reqs.values()):
        assert list(g.token_ids) == _plain_greedy("mixed", prompt, 10), prompt
    eng.manager.check()
    assert not eng.manager.live()


def test_command_line_and_trace_replay(gpu, tmp_path):
    folder, raw, _ = model("wide")
    prompt = util.rand_tokens(9, raw["vocab"], 3)
    p = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--prompt-ids",
                        ",".join(map(str, prompt)), "--dump-tokens", "-n", "6", "--dtype", "fp32", "--temp", "0"],
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [int(x) for x in p.stdout.split()] == _plain_greedy("wide", prompt, 6)
    q = subprocess.run([sys.executable, os.path.join(util.ROOT, "bin", "tuff"), "--model", folder, "--inspect"],
                       capture_output=True, text=True, timeout=300)
    assert q.returncode == 0 and "WkvMixer" in q.stdout and "GatedDeltaMixer" in q.stdout, q.stderr[-2000:]
    # the trace runner: a mixed plan through a child process, four slots, a pool no larger than the plan's peak
    import json
    import numpy as np
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
            rows = [fed[e["id"]] + w for w in e["want"]]
            util.assert_close_f32(data[i:i + len(rows)], want[rows], f"step {s['step']} {e['id']}")
            i += len(rows)
            fed[e["id"]] += len(e["tokens"])
