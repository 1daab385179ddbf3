"""Sovutar on the GPU against the plain implementation (`plain_sovutar.py`): every mechanism alone as the part the
engine runs, in cuts of every size, and whole models through `Engine.step`, the scheduler and `LLM.generate`.

Tolerances.  float32: 2e-5 of the largest plain logit for whole models, 5e-5 of the largest plain output for a
mechanism alone (the plain side is float64; the engine adds in 32 bits).  bfloat16: 3e-2 of the largest plain logit
for whole models, 2.5e-2 of the largest plain output for a mechanism alone.

A router that chooses some of its experts decides by comparing numbers; where two of them lie closer than the
rounding of the layers in front, the plain side and a bfloat16 engine may choose differently, and both are right.
So bfloat16 compares whole models only where every expert is chosen; the choice itself is tested in bfloat16 on the
mixture alone, with inputs that bfloat16 holds exactly, and in whole models in float32.
"""
import pytest
import torch

import plain_sovutar as plain
import replay
from arle_amd import LLM
from arle_amd.cache import CacheManager
from arle_amd.engine import Engine, StepEntry
from arle_amd.engine.batch import build_step_batch
from arle_amd.kernels import ops
from arle_amd.parts import PartSpec
from arle_amd.parts.base import Runtime, build_part
from tiny import random_tokens, read_folder
from tiny_sovutar import NO_CLOSE_CALLS, TINY, chunked, latent, make_model_dir

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: 5e-5, BF16: 2.5e-2}


def rnd(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(BF16).float()     # values that bfloat16 holds exactly


def close(got, want, dtype, what, tol=None):
    got, want = got.double().cpu(), want.double()
    assert torch.isfinite(got).all(), what
    err = float((got - want).abs().max()) / float(want.abs().max())
    assert err <= (tol or TOL[dtype]), f"{what}: {err:.3e}"


def make_part(role, kind, params, tensors, dtype, weights=None):
    rt = Runtime(device=torch.device(DEV), act_dtype=dtype)
    held = {k: v.to(DEV, dtype) for k, v in tensors.items()}
    return build_part(role, PartSpec(kind, params, weights or {k: k for k in tensors}), held.__getitem__, rt)


def run_mixers(parts, x, cuts, *, page=4, dtype=F32):
    """Feed x [T, W] of one request to mixers that run one after the other on the same rows (each with a cache of its
    own, all in one pass, so that one can hand its values to the next) in portions of the given sizes (repeating),
    through a cache in which another request's pages and slot lie between and every page starts as NaN.  Returns the
    concatenated outputs of each part."""
    T = x.shape[0]
    cache = CacheManager([p.cache_need() for p in parts], page_size=page, num_pages=2 * (-(-T // page)) + 4, max_slots=3,
                         max_request_tokens=T + page, device=torch.device(DEV), dtype=dtype)
    cache.admit("other")
    cache.append([("other", page + 1)])
    for group in cache.page_buffers:
        for t in group.values():
            t.fill_(float("nan"))
    cache.admit("r")
    outs, at, k = [[] for _ in parts], 0, 0
    xd = x.to(DEV, dtype)
    while at < T:
        n = min(cuts[k % len(cuts)], T - at)
        k += 1
        before = cache.length("r")
        cache.append([("r", n)])
        cache.sync_tables()
        batch = build_step_batch([StepEntry("r", [0] * n, [])], cache.slot_of.__getitem__, lambda _r, b=before: b, 10, DEV)
        for i, p in enumerate(parts):
            y = p.forward(xd[at:at + n].contiguous(), batch, cache.view(i))
            outs[i].append((y.float().sum(0) if y.dim() == 3 else y.float()).cpu())
        cache.trim_windows("r")
        at += n
    cache.check()
    return [torch.cat(o) for o in outs]


CUTS = [(1000,), (1,), (2,), (5, 2, 7, 3, 1, 16, 2)]


# ----------------------------------------------------------------------------------- mechanisms alone

@pytest.mark.parametrize("dtype", [F32, BF16])
def test_the_norm_on_a_sublayer_s_output_adds_into_the_residual(dtype):
    for width, rows in ((72, 5), (1000, 3), (4100, 2)):
        res = rnd((rows, width), 1, 3.0) + 2.0
        a = rnd((rows, width), 2)
        stack = rnd((3, rows, width), 3)
        outs, wts = rnd((rows, 4, width), 4), rnd((rows, 4), 5).abs()
        w = rnd((width,), 6, 0.2)
        part = make_part("norm", "rmsnorm", {"width": width, "eps": 1e-5, "one_plus": True}, {"weight": w}, dtype)
        for what, terms, total in (
                ("a tensor", a.to(DEV, dtype), a.double()),
                ("a stack", stack.to(DEV), stack.double().sum(0)),
                ("weighted outputs and a stack", [(outs.to(DEV), wts.to(DEV)), stack.to(DEV)],
                 (outs.double() * wts.double()[:, :, None]).sum(1) + stack.double().sum(0))):
            r = res.to(DEV)
            rounded = part.add_into(r, terms)
            want = res.double() + plain.one_plus_norm(total, w.double(), 1e-5)
            close(r, want, F32, f"the residual after {what}, width {width}")
            assert rounded.dtype == dtype
            close(rounded, want, dtype, f"its copy in the activation type after {what}")
            if dtype == F32:
                assert rounded is r
        # the final norm: the same weight kind on the residual itself, on picked rows
        picked = part.add_norm(res.to(DEV), None, rows=torch.tensor([rows - 1, 0], dtype=torch.int32, device=DEV))
        close(picked, plain.one_plus_norm(res.double(), w.double(), 1e-5)[[rows - 1, 0]], dtype, "picked rows")


def chunked_params(width, m, role=None):
    return {"hidden_size": width, "num_q_heads": m["heads"], "num_kv_heads": m["kv_heads"], "key_dim": m["dim"],
            "value_dim": m["vdim"], "qk_norm": True, "eps": 1e-5, "scale": m["scale"],
            "chunk": m["mask"]["size"] if m.get("mask") else None, "window": None, "value_mix": role}


def chunked_tensors(width, m, seed, mix=None):
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t = {"q": rnd((H * D, width), seed, 0.3), "k": rnd((G * D, width), seed + 1, 0.3), "v": rnd((G * Dv, width), seed + 2, 0.3),
         "o": rnd((width, H * Dv), seed + 3, 0.3), "q_norm": 1 + rnd((H * D,), seed + 4, 0.3),
         "k_norm": 1 + rnd((G * D,), seed + 5, 0.3)}
    if mix is not None:
        t["mix"] = torch.tensor(mix).to(BF16).float()
    return t


def plain_names(t):
    return {"q": t["q"].double(), "k": t["k"].double(), "v": t["v"].double(), "o": t["o"].double(),
            "q.norm": t["q_norm"].double(), "k.norm": t["k_norm"].double(),
            "vmix": t["mix"].double() if "mix" in t else None}


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m,page", [(chunked(6, 2, 16, 24, chunk=11), 4), (chunked(4, 4, 32, 8, chunk=8), 8),
                                    (chunked(4, 2, 64, 64, chunk=40), 16), (chunked(5, 1, 24, 40, chunk=21), 16),
                                    (chunked(2, 1, 16, 16, chunk=1), 4), (chunked(3, 1, 8, 16, chunk=None), 4)])
def test_chunked_attention_sees_its_own_chunk_in_every_cut(dtype, m, page):
    width, T = 56, 90
    chunk = m["mask"]["size"] if m.get("mask") else None
    t = chunked_tensors(width, m, 11)
    x = rnd((T, width), 21)
    # a token whose value dwarfs the others right behind a chunk's and a page's border: a mask that is one off shows
    for p in ((chunk or 16), 2 * (chunk or 16) - 1, page * 3):
        if p < T:
            x[p] *= 25.0
    part = make_part("mixer", "wide_norm_attention", chunked_params(width, m), t, dtype)
    want, _ = plain.chunked_attention(x.double(), plain_names(t), m, 1e-5, None)
    first = None
    for cuts in CUTS + [((chunk or 7),), ((chunk or 7) + 1, 1), (page, page + 1)]:
        got, = run_mixers([part], x, cuts, page=page, dtype=dtype)
        close(got, want, dtype, f"chunked attention {m}, cuts {cuts}")
        if dtype == F32:
            first = got if first is None else first
            assert torch.equal(got, first), f"cuts {cuts} change the bits"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_values_are_mixed_with_those_of_the_first_such_layer_and_cached_mixed(dtype):
    width, T = 48, 60
    a, b = chunked(4, 2, 16, 24, chunk=13), chunked(6, 2, 8, 24, chunk=20, scale=0.6)
    ta, tb = chunked_tensors(width, a, 31), chunked_tensors(width, b, 41, mix=0.625)
    x = rnd((T, width), 51)
    x[14] *= 20.0
    source = make_part("mixer", "wide_norm_attention", chunked_params(width, a, "source"), ta, dtype)
    mixer = make_part("mixer", "wide_norm_attention", chunked_params(width, b, "mix"), tb, dtype)
    want_a, v_first = plain.chunked_attention(x.double(), plain_names(ta), a, 1e-5, None)
    want_b, _ = plain.chunked_attention(x.double(), plain_names(tb), b, 1e-5, v_first)
    unmixed, _ = plain.chunked_attention(x.double(), plain_names(tb), b, 1e-5, None)
    assert float((want_b - unmixed).abs().max()) > 0.05 * float(want_b.abs().max())    # leaving the mixing out would show
    for cuts in CUTS:
        got_a, got_b = run_mixers([source, mixer], x, cuts, dtype=dtype)
        close(got_a, want_a, dtype, f"the source layer, cuts {cuts}")
        close(got_b, want_b, dtype, f"the mixing layer, cuts {cuts}")


def test_a_far_key_among_hundreds_is_found_by_the_chunked_attention():
    # q and k read the first half of the input through the same matrix, v reads the second half: a row whose first half
    # repeats an early row's has one score that stands out, and that row's value is the output
    width, T, far = 64, 300, 7
    m = chunked(2, 2, 16, 16, chunk=None, scale=8.0)
    t = chunked_tensors(width, m, 61)
    t["q"][:, 32:] = 0
    t["k"] = t["q"].clone()
    t["q_norm"] = torch.ones_like(t["q_norm"])
    t["k_norm"] = torch.ones_like(t["k_norm"])
    t["v"][:, :32] = 0
    x = rnd((T, width), 71)
    x[T - 1, :32] = x[far, :32]
    x[far, 32:] *= 10.0
    for dtype in (F32, BF16):
        part = make_part("mixer", "wide_norm_attention", chunked_params(width, m), t, dtype)
        want, _ = plain.chunked_attention(x.double(), plain_names(t), m, 1e-5, None)
        for cuts in ((1000,), (T - 1, 1), (64, 3)):
            got, = run_mixers([part], x, cuts, page=16, dtype=dtype)
            close(got[-1:], want[-1:], dtype, f"the last row, cuts {cuts}, {dtype}")


def latent_params(width, m, sink=True):
    return {"hidden_size": width, "heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "value_dim": m["vdim"],
            "rank": m["kv_rank"], "eps": 1e-5, "scale": m["scale"], "window": m["mask"]["size"] if m.get("mask") else None,
            "sink": sink, "position": PartSpec("rope_interleaved", {"head_dim": m["rot_dim"], "rotary_dim": m["rot"]["dims"],
                                                                    "theta": m["rot"]["base"], "max_positions": 1})}


def latent_tensors(width, m, seed):
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    return {"q": rnd((H * (D + R), width), seed, 0.3), "dkv": rnd((C + R, width), seed + 1, 0.3),
            "c_norm": 1 + rnd((C,), seed + 2, 0.3), "uk": rnd((H * D, C), seed + 3, 0.3), "uv": rnd((H * Dv, C), seed + 4, 0.3),
            "sink": rnd((H,), seed + 5) + 1.5, "o": rnd((width, H * Dv), seed + 6, 0.3)}


def plain_latent_names(t):
    return {"q": t["q"].double(), "dkv": t["dkv"].double(), "dkv.norm": t["c_norm"].double(), "uk": t["uk"].double(),
            "uv": t["uv"].double(), "sink": t["sink"].double(), "o": t["o"].double()}


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("m,page", [(latent(3, 24, 8, 20, 40, window=9), 4), (latent(1, 8, 12, 16, 24, window=1, dims=6), 8),
                                    (latent(4, 32, 32, 32, 96, window=37), 16), (latent(20, 16, 16, 16, 48, window=70), 16),
                                    (latent(5, 12, 8, 28, 72, window=19, base=300.0), 16), (latent(2, 8, 4, 8, 16, window=None), 4),
                                    (latent(3, 16, 64, 16, 192, window=45), 16), (latent(18, 8, 16, 8, 144, window=33), 16),
                                    (latent(2, 16, 64, 16, 512, window=30, scale=0.05), 16)])
def test_latent_attention_keeps_its_window_and_its_sink_in_every_cut(dtype, m, page):
    width, T = 56, 100
    window = m["mask"]["size"] if m.get("mask") else None
    t = latent_tensors(width, m, 111)
    x = rnd((T, width), 121)
    # tokens whose rotated key part dwarfs the others': their scores stand out in every head, with either sign, so a
    # window that is one off, or a rotation at the wrong position, shows (less so in bfloat16, where the rounding of a
    # score grows with it: at twelve times the fixed-order kernel on bfloat16 operands is off by 4e-2 as well)
    for p in (3, 2 * page + 1, 50):
        x[p] *= 12.0 if dtype == F32 else 2.0
    part = make_part("mixer", "latent_attention", latent_params(width, m), t, dtype)
    part.prepare(T + 8)
    want = plain.latent_attention(x.double(), plain_latent_names(t), m, 1e-5)
    without = dict(plain_latent_names(t), sink=torch.full((m["heads"],), -1e9, dtype=torch.float64))
    assert float((plain.latent_attention(x.double(), without, m, 1e-5) - want).abs().max()) > 0.02 * float(want.abs().max())
    first = None
    for cuts in CUTS + [((window or 7),), ((window or 7) + 1, 1), (page, page + 1)]:
        got, = run_mixers([part], x, cuts, page=page, dtype=dtype)
        close(got, want, dtype, f"latent attention {m}, cuts {cuts}")
        if dtype == F32:
            first = got if first is None else first
            assert torch.equal(got, first), f"cuts {cuts} change the bits"


def moe_part(width, experts, top, ff, shared, scale, dtype, seed):
    t = {"router": rnd((experts, width), seed, 0.5), "correction": rnd((experts,), seed + 1, 0.3)}
    names = {"router": "router", "correction": "correction"}
    for e in range(experts):
        t.update({f"e{e}.gate": rnd((ff, width), seed + 10 * e + 2, 0.2), f"e{e}.up": rnd((ff, width), seed + 10 * e + 3, 0.2),
                  f"e{e}.down": rnd((width, ff), seed + 10 * e + 4, 0.2)})
        names.update({f"gate{e}": f"e{e}.gate", f"up{e}": f"e{e}.up", f"down{e}": f"e{e}.down"})
    params = {"hidden_size": width, "experts": experts, "top": top, "expert_size": ff, "scale": scale, "correction": True,
              "shared_size": shared, "shared_weights": {"gate": "shared.gate", "up": "shared.up", "down": "shared.down"}}
    if shared:
        t.update({"shared.gate": rnd((shared, width), seed + 5, 0.2), "shared.up": rnd((shared, width), seed + 6, 0.2),
                  "shared.down": rnd((width, shared), seed + 7, 0.2)})
    return make_part("feed_forward", "sigmoid_moe", params, t, dtype, weights=names), t


def moe_sum(terms):
    total = 0      # on the CPU and in a written-out order, so that a row's sum does not depend on the tensor's shape
    for term in terms:
        if isinstance(term, tuple):
            outs, weights = term[0].double().cpu(), term[1].double().cpu()
            for k in range(outs.shape[1]):
                total = total + outs[:, k] * weights[:, k, None]
        else:
            parts = term.double().cpu()
            for part in (parts if parts.dim() == 3 else [parts]):
                total = total + part
    return total


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("experts,top,ff,shared,rows", [(5, 2, 40, 56, 37), (3, 1, 16, None, 9), (4, 4, 24, 32, 70),
                                                        (70, 3, 12, 20, 150), (8, 3, 64, 16, 1), (130, 64, 8, 8, 5)])
def test_the_mixture_chooses_by_corrected_scores_and_weighs_by_the_scores_alone(dtype, experts, top, ff, shared, rows):
    width = 48
    part, t = moe_part(width, experts, top, ff, shared, 1.7, dtype, 200 + experts)
    x = rnd((rows, width), 300 + rows)
    mlp = {"router": {"experts": experts, "top": top, "scale": 1.7}, "shared": {"ff": shared} if shared else None}
    want = plain.moe(x.double(), {k: v.double() for k, v in t.items()}, mlp)
    # the correction changes who is chosen, and must not enter the weights
    uncorrected = plain.moe(x.double(), dict({k: v.double() for k, v in t.items()}, correction=torch.zeros(experts).double()), mlp)
    if top < experts:
        assert float((uncorrected - want).abs().max()) > 0.02 * float(want.abs().max())
    got = moe_sum(part.forward(x.to(DEV, dtype)))
    close(got, want, dtype, f"mixture of {experts} experts, {top} chosen")
    if dtype == F32:    # a row alone is the same bits as in the batch
        for r in (0, rows // 2, rows - 1):
            alone = moe_sum(part.forward(x[r:r + 1].to(DEV, dtype)))
            assert torch.equal(alone[0], got[r])


def test_capped_logits():
    head = make_part("head", "linear", {"vocab_size": 50, "hidden_size": 32, "softcap": 3.0}, {"weight": rnd((50, 32), 1)}, F32)
    x = rnd((7, 32), 2)
    z = x.double() @ rnd((50, 32), 1).double().T
    close(head.forward(x.to(DEV)), 3.0 * torch.tanh(z / 3.0), F32, "capped logits")


# ----------------------------------------------------------------------------------- whole models

@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("sovutar")
    return {name: make_model_dir(base, name) for name in TINY}


def requests_for(cfg, lengths, seed):
    return {f"r{i}": random_tokens(n, cfg["vocab"], seed + i) for i, n in enumerate(lengths)}


def engine_for(folder, name, dtype, tokens, slots=4, **kw):
    return Engine.from_folder(folder, dtype=dtype, page_size=TINY[name][1], max_tokens=tokens, max_slots=slots, **kw)


def references(cfg, weights, reqs):
    return {rid: plain.forward(cfg, weights, toks) for rid, toks in reqs.items()}


MODEL_TOL = {"float32": 2e-5, "bfloat16": 3e-2}


def row_limits(cfg, weights, reqs, ref):
    """What rounding may do to each row in bfloat16.  Every sublayer's output is divided by its own size before it is
    added, so where a sublayer's terms nearly cancel, the rounding of the layers in front is magnified, row by row
    differently (the fixed-order kernels on bfloat16 operands and the matrix-core kernels are off by the same amount
    at the same rows).  A row's limit is five times what changing every matrix entry by up to 2^-9 of itself does to
    the plain logits of that row, and no less than the usual tolerance."""
    limits = {rid: torch.full((len(toks),), MODEL_TOL["bfloat16"], dtype=torch.float64) for rid, toks in reqs.items()}
    for trial in range(2):
        g = torch.Generator().manual_seed(1000 + trial)
        moved = {k: (v * (1 + (torch.rand(v.shape, generator=g) - 0.5) * 2.0 ** -8) if v.dim() == 2 else v)
                 for k, v in weights.items()}
        for rid, toks in reqs.items():
            err = (plain.forward(cfg, moved, toks) - ref[rid]).abs().max(1).values / ref[rid].abs().max()
            limits[rid] = torch.maximum(limits[rid], 5.0 * err)
    return limits


def check_within(got, ref, limits, what):
    errors = []
    for rid, want in ref.items():
        scale = float(want.abs().max())
        for p in range(want.shape[0]):
            row = got[(rid, p)].double()
            assert torch.isfinite(row).all(), f"{what}: non-finite logits at {rid}:{p}"
            err = float((row - want[p]).abs().max()) / scale
            errors.append(err)
            assert err <= float(limits[rid][p]), f"{what}: row {rid}:{p} is off by {err:.3e}, its limit is {float(limits[rid][p]):.3e}"
    assert sorted(errors)[len(errors) // 2] <= MODEL_TOL["bfloat16"], f"{what}: the median row is off by more than the tolerance"


CASES = [(name, dtype) for name in TINY for dtype in ("float32", "bfloat16") if dtype == "float32" or name in NO_CLOSE_CALLS]


@pytest.mark.parametrize("name,dtype", CASES)
def test_whole_prompts_decoding_and_portions_equal_the_plain_logits(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (1, 2, 23, 61, 130), 100)
    ref = references(cfg, weights, reqs)
    eng = engine_for(folders[name], name, dtype, 160)
    limits = row_limits(cfg, weights, reqs, ref) if dtype == "bfloat16" else None
    for how, make in (("whole", replay.whole), ("decode", lambda r, t: replay.prefill_then_decode(r, t, tail=80)),
                      ("portions", replay.portions), ("pairs", lambda r, t: replay.portions(r, t, sizes=(2,))),
                      ("single tokens", lambda r, t: replay.portions(r, t, sizes=(1,)))):
        got = {}
        for rid, toks in reqs.items():
            got.update(replay.run_steps(eng, make(rid, toks)))
        if dtype == "bfloat16":
            check_within(got, ref, limits, f"sovutar {name} {dtype} {how}")
        else:
            replay.check_rows(got, ref, MODEL_TOL[dtype], f"sovutar {name} {dtype} {how}", outlier_tol=8.0)


@pytest.mark.parametrize("name,dtype", CASES)
def test_mixed_batches_with_pages_and_slots_used_again(folders, name, dtype):
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (40, 7, 75, 2, 33, 58, 19, 90), 210)
    ref = references(cfg, weights, reqs)
    # three slots and a pool that just holds the three longest live requests: every slot and page is used again
    eng = engine_for(folders[name], name, dtype, 90 + 75 + 58 + 3 * TINY[name][1], slots=3)
    alone = engine_for(folders[name], name, dtype, 128, slots=1)
    limits = row_limits(cfg, weights, reqs, ref) if dtype == "bfloat16" else None
    for seed in (1, 2):
        steps = replay.mixed(reqs, max_live=3, seed=seed, decode_tail=12, max_portion=17)
        got = replay.run_steps(eng, steps)
        if dtype == "bfloat16":
            check_within(got, ref, limits, f"sovutar {name} {dtype} mixed {seed}")
        else:
            replay.check_rows(got, ref, MODEL_TOL[dtype], f"sovutar {name} {dtype} mixed {seed}", outlier_tol=8.0)
        assert eng.cache.free_slot_count == 3 and eng.cache.free_tokens() == eng.cache.pool_tokens()
    if dtype == "float32":      # in 32 bits a row is the same bits in a batch and alone
        for rid in ("r0", "r3", "r5"):
            solo = replay.run_steps(alone, replay.whole(rid, reqs[rid]))
            for key, row in solo.items():
                assert torch.equal(row, got[key]), f"{key} differs between the batch and the request alone"


@pytest.mark.parametrize("name", ["P", "R"])
def test_bfloat16_rows_do_not_depend_on_the_cut_or_the_batch_beyond_rounding(folders, name):
    # against the engine's own whole-prompt logits, so that a router's close call is the same call on both sides
    # unless the cut itself changes a number
    cfg, weights = read_folder(folders[name])
    reqs = requests_for(cfg, (33, 58, 90, 12), 500)
    eng = engine_for(folders[name], name, "bfloat16", 90 + 58 + 33 + 12 + 64)
    limits = row_limits(cfg, weights, reqs, references(cfg, weights, reqs))
    ref = {}
    for rid, toks in reqs.items():
        rows = replay.run_steps(eng, replay.whole(rid, toks))
        ref[rid] = torch.stack([rows[(rid, p)] for p in range(len(toks))]).double()
    ways = {"decode": sum((replay.prefill_then_decode(r, t, tail=40) for r, t in reqs.items()), []),
            "portions": sum((replay.portions(r, t) for r, t in reqs.items()), []),
            "mixed": replay.mixed(reqs, max_live=4, seed=3, decode_tail=12, max_portion=17)}
    for how, steps in ways.items():
        got = replay.run_steps(eng, steps)
        flipped = 0
        for rid, want in ref.items():
            scale = float(want.abs().max())
            for p in range(want.shape[0]):
                err = float((got[(rid, p)].double() - want[p]).abs().max()) / scale
                flipped += err > float(limits[rid][p])
        total = sum(len(t) for t in reqs.values())
        assert flipped <= (0 if name in NO_CLOSE_CALLS else 0.05 * total), f"{name} {how}: {flipped} of {total} rows differ"


def test_pages_behind_a_chunk_and_a_window_go_back_while_the_request_runs(folders):
    from arle_amd.cache import FREED

    cfg, weights = read_folder(folders["P"])
    toks = random_tokens(61, cfg["vocab"], 77)
    eng = engine_for(folders["P"], "P", "float32", 128)
    got = replay.run_steps(eng, [{"entries": [("a", toks[:57], list(range(57)))], "end": []}])
    page = TINY["P"][1]
    held = {}
    for group in eng.cache.groups:
        pages = group.tables["a"].pages
        held[(group.window, group.chunk)] = sum(p != FREED for p in pages)
        if group.chunk:      # every page in front of the chunk that position 57 falls into has gone back
            assert all(p == FREED for p in pages[:(57 // group.chunk * group.chunk) // page])
    assert held[(None, 11)] == -(-57 // page) - 55 // page and held[(None, 30)] == -(-57 // page) - 30 // page
    assert held[(9, None)] == -(-57 // page) - (57 - 9 + 1) // page
    for i in range(57, 61):      # and what follows still equals the plain logits
        got.update(replay.run_steps(eng, [{"entries": [("a", toks[i:i + 1], [0])], "end": ["a"] if i == 60 else []}]))
    replay.check_rows(got, {"a": plain.forward(cfg, weights, toks)}, MODEL_TOL["float32"], "after pages went back")


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
        toks.append(int(plain.forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


@pytest.mark.parametrize("name", ["P", "S"])
def test_greedy_generation_through_the_scheduler_equals_the_plain_implementation(folders, name):
    cfg, weights = read_folder(folders[name])
    prompts = [random_tokens(n, cfg["vocab"], 400 + n) for n in (3, 12, 29, 18, 7)]
    want = [_plain_greedy(cfg, weights, p, 24) for p in prompts]
    # two slots for five requests, portions of at most eight tokens: slots and pages are used again
    llm = LLM(folders[name], dtype="float32", page_size=TINY[name][1], kv_cache_tokens=160, max_seq_len=64, num_slots=2,
              chunked_prefill_size=8)
    outs = llm.generate(prompts, max_tokens=24)
    assert [o.response_token_ids for o in outs] == want
    assert all(o.finish_reason == "length" for o in outs)
