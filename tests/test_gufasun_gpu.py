"""Gufasun on the GPU against the plain implementation (`plain_gufasun.py`): every mechanism alone as the part
the engine runs, in cuts of every size, and whole models through `Engine.step`, the scheduler and `LLM.generate`.

Tolerances.  float32: 2e-5 of the largest plain logit for whole models, 5e-5 of the largest plain output for a
mechanism alone, where a token is made to stand out on purpose (the plain side is float64; the engine adds in 32 bits;
measured 3e-7 to 4e-5).
bfloat16: 3e-2 of the largest plain logit for whole models, a bound on rounding through a few layers; the
mechanisms alone are held to 2.5e-2 of their largest plain output.
"""
import pytest
import torch

import plain_gufasun as plain
import replay
from arle_amd import LLM
from arle_amd.cache import CacheManager
from arle_amd.engine import Engine, StepEntry
from arle_amd.engine.batch import build_step_batch
from arle_amd.parts import PartSpec
from arle_amd.parts.base import Pending, Runtime, build_part
from arle_amd.parts.short_conv import InputConvMixer
from tiny import random_tokens, read_folder
from tiny_gufasun import TINY, attention, make_model_dir, mlstm

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 5e-5, BF16: 2.5e-2}


def rnd(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(BF16).float()     # values that bfloat16 holds exactly


def close(got, want, dtype, what):
    got, want = got.double().cpu(), want.double()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max()) / float(want.abs().max())
    assert err <= TOL[dtype], f"{what}: {err:.3e}"


def make_part(role, kind, params, tensors, dtype):
    rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    held = {k: v.to(DEV, dtype) for k, v in tensors.items()}
    return build_part(role, PartSpec(kind, params, {k: k for k in tensors}), held.__getitem__, rt)


def run_mixer(part, x, cuts, *, page=4, slot_noise=True, readers=None, owner=None, dtype=F32):
    """Feed x [T, W] of one request to a mixer in portions of the given sizes (repeating), through a cache of its
    own in which another request's pages and slot lie between; returns the concatenated outputs.  `owner`: a part
    that runs before it on the same rows and whose pages it reads."""
    parts = [owner, part] if owner is not None else [part]
    needs = [p.cache_need() for p in parts]
    T = x.shape[0]
    cache = CacheManager(needs, page_size=page, num_pages=2 * (-(-T // page)) + 4, max_slots=3, max_request_tokens=T + page,
                         device=torch.device(DEV), dtype=dtype, readers={1: 0} if owner is not None else None)
    if slot_noise:      # slot 0 and the first pages belong to somebody else, and every state starts as rubbish
        cache.admit("other")
        cache.append([("other", page + 1)])
        for buf in cache.state_buffers.values():
            buf.fill_(float("nan"))
        for group in cache.page_buffers:
            for t in group.values():
                t.fill_(float("nan"))
    cache.admit("r")
    outs, at, k = [], 0, 0
    xd = x.to(DEV, dtype)
    while at < T:
        n = min(cuts[k % len(cuts)], T - at)
        k += 1
        before = cache.length("r")
        cache.append([("r", n)])
        cache.sync_tables()
        batch = build_step_batch([StepEntry("r", [0] * n, [])], cache.slot_of.__getitem__, lambda _r, b=before: b, 10, DEV)
        y = None
        for i, p in enumerate(parts):
            y = p.forward(xd[at:at + n].contiguous(), batch, cache.view(i))
        y = y[0] if isinstance(y, tuple) else y
        outs.append((y.float().sum(0) if y.dim() == 3 else y.float()).cpu())
        cache.trim_windows("r")
        at += n
    cache.check()
    return torch.cat(outs)


CUTS = [(1000,), (1,), (2,), (5, 2, 7, 3, 1, 16, 2)]


# ----------------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("dtype", [F32, BF16])
def test_layer_norm_adds_what_is_pending_and_gives_two_norms_from_one_pass(dtype):
    for width, rows in ((72, 5), (1000, 3), (1024 + 8, 2), (5000, 2)):
        res = rnd((rows, width), 1, 3.0) + 2.0
        a, b = rnd((rows, width), 2).to(dtype).float(), rnd((3, rows, width), 3)
        ba, bb = rnd((width,), 4), rnd((width,), 5)
        w1, w2 = 1 + rnd((width,), 6, 0.1), 1 + rnd((width,), 7, 0.1)
        part = make_part("norm", "layernorm", {"width": width, "eps": 1e-5}, {"weight": w1}, dtype)
        other = make_part("norm", "layernorm", {"width": width, "eps": 1e-5}, {"weight": w2}, dtype)
        r = res.to(DEV)
        pending = Pending([(a.to(DEV, dtype), ba.to(DEV, dtype)), (b.to(DEV), bb.to(DEV, dtype))])
        o1, o2 = part.add_norm(r, pending, also=other)
        total = res.double() + a.double() + ba.double() + b.double().sum(0) + bb.double()
        close(r, total, F32, "the residual after the add")
        close(o1, plain.layer_norm(total, w1.double(), 1e-5), dtype, f"first norm, width {width}")
        close(o2, plain.layer_norm(total, w2.double(), 1e-5), dtype, f"second norm, width {width}")
        rows_wanted = torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEV)
        kept = r.clone()
        picked = part.add_norm(r, a.to(DEV, dtype), rows=rows_wanted)
        assert torch.equal(r, kept)                      # with rows named the sum is not written back
        close(picked, plain.layer_norm((total + a.double())[[rows - 1, 0]], w1.double(), 1e-5), dtype, "picked rows")


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_input_convolution_is_the_same_in_every_cut(dtype, taps):
    class Through:
        graph_safe = True
        def cache_need(self): return None
        def forward(self, h, batch, cache): return h
    width, T = 40, 37
    x, w = rnd((T, width), 11), rnd((width, taps), 12, 0.5)
    part = InputConvMixer({"width": width, "taps": taps}, {"weight": w.to(DEV, dtype)},
                          Runtime(torch.device(DEV), dtype), {"inner": Through()})
    want = x.double() + plain.causal_conv(x.double(), w.double())
    first = None
    for cuts in CUTS:
        got = run_mixer(part, x, cuts, dtype=dtype)
        close(got, want, dtype, f"taps {taps}, cuts {cuts}")
        first = got if first is None else first
        assert torch.equal(got, first), f"taps {taps}: cuts {cuts} change the bits"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_polynorm_feed_forward(dtype):
    for width, ff, rows in ((40, 56, 7), (72, 2100, 3), (64, 9000, 2)):
        t = {"up": rnd((ff, width), 21, 0.3), "up_bias": rnd((ff,), 22, 0.3), "down": rnd((width, ff), 23, 0.1),
             "down_bias": rnd((width,), 24), "coef": torch.tensor([0.75, -0.5, 0.25, 0.125])}
        part = make_part("feed_forward", "polynorm", {"hidden_size": width, "intermediate_size": ff, "eps": 1e-5}, t, dtype)
        x = rnd((rows, width), 25)
        y, bias = part.forward(x.to(DEV, dtype))
        got = (y.float().sum(0) if y.dim() == 3 else y.float()) + bias.float()
        d = {k: v.double() for k, v in t.items()}
        want = plain.poly_norm_ffn(x.double(), d["up"], d["up_bias"], d["down"], d["down_bias"], d["coef"], 1e-5)
        close(got, want, dtype, f"ff {ff}")


def mlstm_tensors(width, m, seed, gate_std=0.5):
    """gate_std: spread of the gate projections.  With 0.5 input gates differ by thousands, one token can dominate the
    memory, and where its key is nearly orthogonal to a query the output's sign hangs on the last bits: right for the
    32-bit comparison, which holds there too, but no measure of bfloat16 rounding, which gets 0.05."""
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    return {"q": rnd((H * D, width), seed, 0.3), "k": rnd((H * D, width), seed + 1, 0.3), "v": rnd((H * Dv, width), seed + 2, 0.3),
            "g": rnd((H * Dv, width), seed + 3, 0.3), "o": rnd((width, H * Dv), seed + 4, 0.2), "norm": 1 + rnd((H * Dv,), seed + 5, 0.1),
            "i": rnd((H, width), seed + 6, gate_std), "i_bias": rnd((H,), seed + 7), "f": rnd((H, width), seed + 8, gate_std),
            "f_bias": rnd((H,), seed + 9) + 5.0}      # forget gates near one: what token 4 left is still there at the end


def plain_names(t):
    return {k.replace("_bias", ".b").replace("_conv", ".conv").replace("_norm", ".norm"): v.double() for k, v in t.items()}


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m", [mlstm(3, 12, 20), mlstm(1, 64, 100, cap=3.0), mlstm(2, 130, 70), mlstm(2, 8, 8, cap=12.0)])
def test_mlstm_in_every_cut_and_over_a_long_sequence(dtype, m):
    width, T = 48, 150
    t = mlstm_tensors(width, m, 31, gate_std=0.5 if dtype == F32 else 0.05)
    x = rnd((T, width), 41)
    # one early token that the memory has to keep: its value stands out for the rest of the sequence (in bfloat16 by
    # less: a token that dominates makes the output's direction hang on the sign of single dot products)
    x[4] *= 12.0 if dtype == F32 else 1.5
    params = {"hidden_size": width, "heads": m["heads"], "key_dim": m["dim"], "value_dim": m["vdim"],
              "gate_cap": m["gate_cap"], "eps": 1e-5}
    part = make_part("mixer", "mlstm", params, t, dtype)
    want = plain.mlstm_mixer(x.double(), plain_names(t), m, 1e-5)
    first = None
    for cuts in CUTS:
        got = run_mixer(part, x, cuts, dtype=dtype)
        close(got, want, dtype, f"mlstm {m}, cuts {cuts}")
        if dtype == F32:        # in 32 bits a row's sums run in one order however the sequence is cut
            first = got if first is None else first
            assert torch.equal(got, first), f"cuts {cuts} change the bits"


def attention_tensors(width, m, seed, shares=False):
    H, G, D, Dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
    t = {"q": rnd((H * D, width), seed, 0.3), "q_bias": rnd((H * D,), seed + 1, 0.3), "q_norm": 1 + rnd((D,), seed + 2, 0.1),
         "r1": 0.5 + rnd((H,), seed + 3, 0.1), "r2": 1 + rnd((H,), seed + 4, 0.2), "o": rnd((width, H * Dv), seed + 5, 0.2)}
    if taps:
        t["q_conv"] = rnd((H * D, taps), seed + 6, 0.5)
    if not shares:
        t.update({"k": rnd((G * D, width), seed + 7, 0.3), "k_bias": rnd((G * D,), seed + 8, 0.3),
                  "v": rnd((G * Dv, width), seed + 9, 0.3), "v_bias": rnd((G * Dv,), seed + 10, 0.3),
                  "k_norm": 1 + rnd((D,), seed + 11, 0.1)})
        if taps:
            t.update({"k_conv": rnd((G * D, taps), seed + 12, 0.5), "v_conv": rnd((G * Dv, taps), seed + 13, 0.5)})
    return t


def attention_params(width, m, shares=False, cache_window=None):
    return {"hidden_size": width, "num_q_heads": m["heads"], "num_kv_heads": m["kv_heads"], "key_dim": m["dim"],
            "value_dim": m["vdim"], "bias": True, "conv_taps": m["conv"], "qk_norm": True, "eps": 1e-5,
            "temp_coef": m["q_temp"]["coef"], "temp_every": m["q_temp"]["every"], "scale": m["scale"],
            "softcap": m["softcap"], "distance_penalty": True, "window": m["mask"]["size"],
            "cache_window": cache_window or m["mask"]["size"], "shares_kv": shares}


def plain_attention(x, t, m, kv_from=None):
    p = plain_names(t)
    keys, values = kv_from if kv_from is not None else plain.attention_keys_values(x.double(), p, m, 1e-5)
    return plain.attention_mixer(x.double(), p, m, 1e-5, keys, values), (keys, values)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m, page", [(attention(6, 2, 16, 32, window=7), 4), (attention(2, 2, 32, 24, window=8, conv=0, every=1), 8),
                                     (attention(4, 1, 16, 16, window=1, conv=5), 4), (attention(4, 2, 80, 96, window=40, conv=4, every=16), 16),
                                     (attention(8, 2, 64, 64, window=33, conv=2, softcap=2.0), 16)])
def test_attention_in_every_cut_with_a_value_that_shows_at_the_window_s_edge(dtype, m, page):
    width, T = 56, 90
    window = m["mask"]["size"]
    t = attention_tensors(width, m, 51)
    x = rnd((T, width), 61)
    j = 2 * page + 1       # a key right behind a page border whose value dwarfs the others: it counts for exactly
    x[j] *= 25.0 * max(1, window // 4)   # `window` rows (and, through the convolution, its next taps - 1 neighbours do)
    part = make_part("mixer", "softcap_attention", attention_params(width, m), t, dtype)
    want, _ = plain_attention(x, t, m)
    ref_in, ref_out = want[j + window - 1].abs().max(), want[j + window + max(m["conv"], 1) - 1].abs().max()
    assert ref_in > 1.3 * ref_out     # the plain side does show the edge
    first = None
    for cuts in CUTS + [(window,), (window + 1, 1), (page, page + 1)]:
        got = run_mixer(part, x, cuts, page=page, dtype=dtype)
        close(got, want, dtype, f"attention {m}, cuts {cuts}")
        if dtype == F32:
            first = got if first is None else first
            assert torch.equal(got, first), f"cuts {cuts} change the bits"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_a_layer_reads_another_layer_s_keys_and_values_through_its_own_wider_window(dtype):
    width, T = 56, 70
    own = attention(6, 2, 16, 32, window=5)
    reader = attention(6, 2, 16, 32, window=19, softcap=3.0, every=4, conv=2)
    t_own, t_reader = attention_tensors(width, own, 71), attention_tensors(width, reader, 81, shares=True)
    x = rnd((T, width), 91)
    x[9] *= 25.0
    owner = make_part("mixer", "softcap_attention", attention_params(width, own, cache_window=19), t_own, dtype)
    part = make_part("mixer", "softcap_attention", attention_params(width, reader, shares=True), t_reader, dtype)
    _, kv = plain_attention(x, t_own, own)
    want, _ = plain_attention(x, t_reader, reader, kv_from=kv)
    for cuts in CUTS:
        close(run_mixer(part, x, cuts, owner=owner, dtype=dtype), want, dtype, f"reader, cuts {cuts}")


# ----------------------------------------------------------------------------------- whole models

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("gufasun")
    return {name: make_model_dir(base, name) for name in TINY}


def requests_for(cfg, lengths, seed):
    return {f"r{i}": random_tokens(n, cfg["vocab"], seed + i) for i, n in enumerate(lengths)}


def engine_for(folder, name, dtype, tokens, slots=4, **kw):
    return Engine.from_folder(folder, dtype=dtype, page_size=TINY[name][1], max_tokens=tokens, max_slots=slots, **kw)


def references(cfg, weights, reqs):
    return {rid: plain.forward_logits(weights, cfg, toks) for rid, toks in reqs.items()}


MODEL_TOL = {"float32": 2e-5, "bfloat16": 3e-2}
# A row's rms error against the median row's.  The recurrence's conditioning differs from row to row: where the plain
# logits of a row move 11 times as much as the median row's under a change of 1e-6 in the weights, the engine's error
# in both precisions was 20 times the median's, batched or alone.  Measured on these requests: up to 5 in bfloat16; in
# float32, where every row is held to 2e-5 anyway, up to 15 (a request's first row in a model of matrix memories only).
SPREAD = {"float32": 25.0, "bfloat16": 8.0}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_whole_prompts_decoding_and_portions_equal_the_plain_logits(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (1, 2, 23, 61, 130), 100)
    ref = references(cfg, weights, reqs)
    eng = engine_for(folders[name], name, dtype, 160)
    for how, make in (("whole", replay.whole), ("decode", lambda r, t: replay.prefill_then_decode(r, t, tail=40)),
                      ("portions", replay.portions), ("pairs", lambda r, t: replay.portions(r, t, sizes=(2,))),
                      ("single tokens", lambda r, t: replay.portions(r, t, sizes=(1,)))):
        got = {}
        for rid, toks in reqs.items():
            got.update(replay.run_steps(eng, make(rid, toks)))
        replay.check_rows(got, ref, MODEL_TOL[dtype], f"gufasun {name} {dtype} {how}", outlier_tol=SPREAD[dtype])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(TINY))
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (40, 7, 75, 2, 33, 58, 19, 90), 210)
    ref = references(cfg, weights, reqs)
    # three slots and a pool that just holds the three longest live requests: every slot and page is used again
    eng = engine_for(folders[name], name, dtype, 90 + 75 + 58 + 3 * TINY[name][1], slots=3)
    alone = engine_for(folders[name], name, dtype, 128, slots=1)
    for seed in (1, 2):
        steps = replay.mixed(reqs, max_live=3, seed=seed, decode_tail=12, max_portion=17)
        got = replay.run_steps(eng, steps)
        replay.check_rows(got, ref, MODEL_TOL[dtype], f"gufasun {name} {dtype} mixed {seed}", outlier_tol=SPREAD[dtype])
        assert eng.cache.free_slot_count == 3 and (not eng.cache.groups or eng.cache.free_tokens() == eng.cache.pool_tokens())
    if dtype == "float32":      # in 32 bits a row is the same bits in a batch and alone
        for rid in ("r0", "r3", "r5"):
            solo = replay.run_steps(alone, replay.whole(rid, reqs[rid]))
            for key, row in solo.items():
                assert torch.equal(row, got[key]), f"{key} differs between the batch and the request alone"


def test_captured_steps_give_the_bits_of_eager_ones(folders):
    cfg, _ = read_folder(folders["P"])
    reqs = requests_for(cfg, (30, 30, 41), 300)
    steps = []
    for rid, toks in reqs.items():      # equal portions, then decoding: shapes repeat and are captured
        steps += [{"entries": [(rid, toks[i:i + 6], list(range(len(toks[i:i + 6]))))], "end": []} for i in range(0, 24, 6)]
    live = list(reqs)
    for i in range(24, 30):
        steps.append({"entries": [(rid, reqs[rid][i:i + 1], [0]) for rid in live], "end": live if i == 29 else []})
    out = {}
    for graphs in (False, True):
        eng = engine_for(folders["P"], "P", "bfloat16", 160, cuda_graph=graphs)
        out[graphs] = replay.run_steps(eng, steps)
        assert (eng.graph_replays > 0) == graphs
    assert all(torch.equal(out[True][k], out[False][k]) for k in out[False])


def _plain_greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(plain.forward_logits(weights, cfg, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["P", "R"])
def test_greedy_generation_through_the_scheduler_equals_the_plain_implementation(folders, name):
    cfg, weights = read_folder(folders[name])
    prompts = [random_tokens(n, cfg["vocab"], 400 + n) for n in (3, 12, 29, 18, 7)]
    want = [_plain_greedy(cfg, weights, p, 24) for p in prompts]
    # two slots for five requests, portions of at most eight tokens: slots, pages and states are used again
    llm = LLM(folders[name], dtype="float32", page_size=TINY[name][1], kv_cache_tokens=160, max_seq_len=64, num_slots=2,
              chunked_prefill_size=8)
    outs = llm.generate(prompts, max_tokens=24)
    assert [o.response_token_ids for o in outs] == want
    assert all(o.finish_reason == "length" for o in outs)
