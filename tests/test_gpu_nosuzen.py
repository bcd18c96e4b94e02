"""The Nosuzen decoder in the engine against the plain implementation of tests/plain/nosuzen.py: every mechanism
alone, whole prompts against decoding token by token, portions down to two tokens, mixed batches with pages and
state slots that are used again, keys far back and at the edges of every window, the first positions that a window
keeps, long decoding from recorded graphs, and greedy generation through ``LLM.generate`` and the scheduler; on three
small configurations that differ in every size, in 32-bit and in bfloat16.  The kernels that are new with this design
are also compared alone, on inputs made so that a fault shows."""

import math

import pytest
import torch

from . import nosuzen_models as models
from . import schedules
from .helpers import random_tokens
from .plain import nosuzen as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [70, 41, 100, 35, 50, 33], "B": [66, 40, 130, 35, 90], "C": [45, 150, 37, 64, 120]}
#: distances are measured as a replay of a trace is judged: the difference of two rows of logits with its mean taken
#: off, root mean square over the vocabulary, over the root mean square of the truth
FP32_TOL = 3e-5
BF16_TOL = 5e-2
DEV = "cuda:0"


def distance(got: torch.Tensor, truth: torch.Tensor, scale: float) -> float:
    d = got.double() - truth.double()
    d = d - d.mean()
    return float(d.pow(2).mean().sqrt()) / scale


def truth_of(cfg, weights, requests):
    out = {rid: plain.forward(cfg, weights, toks) for rid, toks in requests.items()}
    scale = float(torch.cat([(t - t.mean(-1, keepdim=True)).flatten() for t in out.values()]).pow(2).mean().sqrt())
    return out, scale


def folder_for(dtype, path, cfg_dict, **kw):
    """The model a run in ``dtype`` is compared on.  Rounding to bfloat16 moves a router's scores a little, and where
    two experts lie closer than that the engine and the plain model choose differently for a token; so bfloat16 runs
    get routers whose choice no rounding changes, and the 32-bit runs, which are the sharp ones, get routers whose
    choice changes from token to token."""
    return models.make_folder(path / dtype, cfg_dict, decisive_router=dtype == "bfloat16", **kw)


def assert_within_rounding(dists, tol, what):
    """bfloat16 against the plain model: all but 5% of the positions lie under the bound, and their mean under half
    of it.  (A few positions stand out, the same in every schedule: a channel of a norm's input near zero under a
    steep tanh, or a head whose two maps nearly cancel before the join divides by their difference's root mean
    square, magnify rounding.)  A fault of a kernel moves every position."""
    d = sorted(dists)
    keep = d[: max(len(d) - max(len(d) * 5 // 100, 1), 1)]
    assert keep[-1] < tol, f"{what}: {sum(x >= tol for x in d)} of {len(d)} positions at or over {tol}, the worst kept {keep[-1]}"
    assert sum(keep) / len(keep) < tol / 2, f"{what}: mean distance {sum(keep) / len(keep)}"


class Case:
    def __init__(self, name, tmp):
        from torchllms_amd.engine import Engine

        self.name = name
        self.folders = {dt: folder_for(dt, tmp / name, models.CONFIGS[name], seed=11) for dt in ("float32", "bfloat16")}
        self.cfg = models.CONFIGS[name]
        self.requests = {f"r{i}": random_tokens(n, self.cfg["vocab"], 100 + i) for i, n in enumerate(LENGTHS[name])}
        self.truths = {dt: truth_of(*models.read_folder(f), self.requests) for dt, f in self.folders.items()}
        self.traces = {
            "whole": schedules.whole(self.requests),
            "tail": schedules.tail(self.requests),
            "portions": schedules.portions(self.requests),
            "mixed": schedules.mixed(self.requests),
        }
        page = models.PAGE_SIZE[name]
        pool_tokens = max(schedules.max_live_tokens(t) for t in self.traces.values())
        self.engines = {
            dt: Engine.from_folder(self.folders[dt], dtype=dt, page_size=page, num_pages=-(-pool_tokens // page), max_seqs=4)
            for dt in ("float32", "bfloat16")
        }
        self._results = {}

    def result(self, dtype, schedule):
        key = (dtype, schedule)
        if key not in self._results:
            self._results[key] = run_trace(self.engines[dtype], self.traces[schedule])
        return self._results[key]

    def distances(self, dtype, result):
        truth, scale = self.truths[dtype]
        return [distance(row, truth[rid][pos], scale) for (rid, pos), row in result.items()]

    def worst(self, result):
        truth, scale = self.truths["float32"]
        worst, where = 0.0, None
        for (rid, pos), row in result.items():
            e = distance(row, truth[rid][pos], scale)
            if not e <= worst:
                worst, where = e, (rid, pos)
        return worst, where


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("nosuzen")
    return {name: Case(name, tmp) for name in models.CONFIGS}


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_matches_the_plain_model(cases, name, schedule):
    case = cases[name]
    got = case.result("float32", schedule)
    assert len(got) == sum(len(t) for t in case.requests.values())
    err, where = case.worst(got)
    assert err < FP32_TOL, f"{name}/{schedule}: first look at {where}, distance {err}"


@pytest.mark.parametrize("schedule", ["tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_does_not_depend_on_the_schedule(cases, name, schedule):
    """Every 32-bit kernel adds in an order fixed by the element it computes (blocks of keys aligned to positions, the
    recurrence token by token, the experts pair by pair in the order of a token's choices, the streams one after the
    other), so cutting, batching, pages and slots change no bit."""
    case = cases[name]
    ref = case.result("float32", "whole")
    got = case.result("float32", schedule)
    diff = sorted(k for k in ref if not torch.equal(ref[k], got[k]))
    assert not diff, f"{name}/{schedule}: {len(diff)} positions differ, first {diff[0]}"


@pytest.mark.parametrize("schedule", ["whole", "tail", "portions", "mixed"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_bfloat16_stays_within_rounding(cases, name, schedule):
    case = cases[name]
    got = case.result("bfloat16", schedule)
    assert_within_rounding(case.distances("bfloat16", got), BF16_TOL, f"{name}/{schedule}")


# ----------------------------------------------------------------------------- every mechanism alone
_R = models.rot
_TINY_MOE = models.moe(8, 2, 1)
ALONE = {
    "differential": models.layer("attention", models.diff_attention(4, 2, 24, 40, 0.2, 0.5, _R(12, 1000.0), 30, keep_first=4, conv=3)),
    "differential_no_conv_no_window_edge": models.layer("attention", models.diff_attention(2, 2, 16, 16, 0.3, 0.1, _R(16, 100.0), 1000)),
    "differential_one_tap_odd_sizes": models.layer("attention", models.diff_attention(3, 1, 20, 36, 0.2, 0.8, _R(0), 19, keep_first=19, conv=1)),
    "differential_wide": models.layer("attention", models.diff_attention(2, 1, 128, 256, 0.08, 0.6, _R(64, 1e6, (4.0, 64, 16.0, 1.0)), 64, keep_first=70, conv=2)),
    "differential_matrix_cores": models.layer("attention", models.diff_attention(4, 2, 64, 128, 0.12, 0.5, _R(64, 1e4, (4.0, 64, 16.0, 1.0)), 50, keep_first=7, conv=2)),
    "differential_matrix_cores_same_width": models.layer("attention", models.diff_attention(2, 1, 128, 128, 0.09, 0.3, _R(32, 1e4), 33, keep_first=40)),
    "latent_matrix_cores": models.layer("latent_attention", models.latent(4, 24, 32, 40, 96, 0.15, 40, scaling=(4.0, 64, 8.0, 1.0))),
    "latent_odd": models.layer("latent_attention", models.latent(3, 20, 6, 28, 50, 0.2, 25, base=50.0)),
    "latent_nothing_rotated_wide_latent": models.layer("latent_attention", models.latent(2, 16, 0, 8, 288, 0.2, 90)),
    "latent_one_key_window": models.layer("latent_attention", models.latent(2, 16, 8, 16, 24, 0.2, 1)),
    # one side of a parallel layer alone: the other's weight is zero
    "softmax_side": models.layer("parallel", models.pair(models.left(4, 2, 24, 40, 0.25, _R(10, 1e4, (4.0, 16, 8.0, 1.0)), 22, keep_first=6), models.right(1, 8, 8, 4.0, 2), 1.3, 0.0)),
    "softmax_side_matrix_cores": models.layer("parallel", models.pair(models.left(8, 2, 64, 64, 0.2, _R(32), 45), models.right(1, 8, 8, 4.0, 2), 1.0, 0.0)),
    "softmax_side_keeps_more_than_its_window": models.layer("parallel", models.pair(models.left(2, 1, 32, 32, 0.2, _R(32), 8, keep_first=33), models.right(1, 8, 8, 4.0, 2), 1.0, 0.0)),
    "linear_side": models.layer("parallel", models.pair(models.left(1, 1, 8, 8, 0.3, _R(0), 5), models.right(4, 24, 40, 12.0, 6), 0.0, 1.2)),
    "linear_side_wide": models.layer("parallel", models.pair(models.left(1, 1, 8, 8, 0.3, _R(0), 5), models.right(1, 256, 64, 64.0, 32), 0.0, 0.7)),
    "linear_side_odd": models.layer("parallel", models.pair(models.left(1, 1, 8, 8, 0.3, _R(0), 5), models.right(3, 18, 70, 1.0, 3), 0.0, 1.0)),
    "both_sides": models.layer("parallel", models.pair(models.left(2, 1, 32, 32, 0.2, _R(32), 16, keep_first=2), models.right(2, 32, 16, 8.0, 8), 0.6, 0.5)),
    "routed_groups": models.layer("latent_attention", models.latent(1, 8, 4, 8, 16, 0.3, 4), models.moe(40, 8, 3, 1.25, groups=(4, 2), shared=56)),
    "routed_one_choice": models.layer("latent_attention", models.latent(1, 8, 4, 8, 16, 0.3, 4), models.moe(33, 5, 1, 0.7)),
    "routed_every_expert_its_own_group": models.layer("latent_attention", models.latent(1, 8, 4, 8, 16, 0.3, 4), models.moe(16, 6, 2, 1.0, groups=(6, 3))),
    "routed_all_chosen": models.layer("latent_attention", models.latent(1, 8, 4, 8, 16, 0.3, 4), models.moe(16, 3, 3, 1.0, groups=(1, 1), shared=8)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("what", sorted(ALONE))
def test_a_mechanism_alone(tmp_path, what, dtype):
    """A model of one layer, a prompt in one step and, in a second request, the same tokens in portions and one by one;
    with one stream, two or three."""
    from torchllms_amd.engine import Engine, StepEntry

    streams = 1 + len(what) % 3
    folder = folder_for(dtype, tmp_path / what, models.single_layer(ALONE[what], streams=streams), seed=5)
    cfg, weights = models.read_folder(folder)
    tokens = random_tokens(275, cfg["vocab"], 9)
    truth, scale = truth_of(cfg, weights, {"r": tokens})
    engine = Engine.from_folder(folder, dtype=dtype, page_size=8, num_pages=80, max_seqs=2)
    engine.admit("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
    engine.admit("cut")
    rows, at = [], 0
    for n in (5, 2, 30, 1, 1, 1, 17, 2, 1, 1, 13, 1, 150, 1, 1, 47, 1):
        rows.append(engine.step([StepEntry("cut", tokens[at : at + n], list(range(n)))]).cpu())
        at += n
        engine.cache.check_invariants()
    assert at == len(tokens)
    cut = torch.cat(rows)
    # (a single layer's output norm divides by a root mean square that a random model lets come near zero at a position
    # or two, where 32-bit rounding shows a hundred times larger, in the plain model too: a position's bound is the
    # usual one, or three times what the plain model run in 32-bit is away from the 64-bit truth there)
    own = plain.forward(cfg, weights, tokens, dtype=torch.float32) if dtype == "float32" else None
    for name, got in (("whole", whole), ("cut", cut)):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(len(tokens))]
        if dtype == "float32":
            over = [(i, d) for i, d in enumerate(dists) if d >= max(FP32_TOL, 3 * distance(own[i], truth["r"][i], scale))]
            assert not over, f"{what}/{name}: {over[:5]}"
        else:
            assert_within_rounding(dists, BF16_TOL, f"{what}/{name}")
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- the new kernels alone
def _paged(keys, values, page, n_pages, gen):
    """Keys [n, Hk, d] and values [n, Hv, dv] of one request in pages handed out in a shuffled order; the pool holds
    other numbers everywhere else.  Returns (k_pages, v_pages, block table row, slots)."""
    n = keys.shape[0]
    order = torch.randperm(n_pages, generator=gen)[: -(-n // page)]
    k_pages = torch.randn((n_pages, keys.shape[1], page, keys.shape[2]), generator=gen) * 3
    v_pages = torch.randn((n_pages, values.shape[1], page, values.shape[2]), generator=gen) * 3
    for j in range(n):
        k_pages[order[j // page], :, j % page] = keys[j]
        v_pages[order[j // page], :, j % page] = values[j]
    return k_pages, v_pages, order.to(torch.int32)


def _plain_attention(q, keys, values, pos, window, keep, scale, group):
    """softmax attention of one query [Hq, d] at position ``pos`` over keys [n, Hk, d] / values [n, Hv, dv]: query head h
    reads key head h // group and value head (h // group) % Hv; it sees j <= pos with pos - j < window or j < keep."""
    out = []
    for h in range(q.shape[0]):
        g = h // group
        js = [j for j in range(pos + 1) if pos - j < window or j < keep]
        s = torch.stack([(q[h].double() * keys[j, g].double()).sum() * scale for j in js])
        p = torch.softmax(s, 0)
        out.append(sum(p[i] * values[j, g % values.shape[1]].double() for i, j in enumerate(js)))
    return torch.stack(out)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("Hq,Hk,Hv,d,dv,page", [(4, 2, 2, 16, 16, 8), (8, 4, 2, 24, 40, 4), (6, 2, 1, 64, 32, 16), (2, 2, 2, 7, 5, 3)])
def test_plain_attention_with_kept_first_keys_and_fewer_value_heads(Hq, Hk, Hv, d, dv, page, dtype):
    """A window of 37 that keeps the first 11 positions, over 300 keys.  Four keys are made to stand out for every
    query: the last one inside the window and the first one outside it, the last kept position and the first that
    is not kept; a mask that is one off at either edge changes the result by much more than the bound.  The same
    queries as single tokens (a wave walks alone), as a prompt's portion (tiles through LDS), as decode steps with
    blocks of keys side by side, and at positions where the kept keys and the window meet or overlap."""
    from torchllms_amd.kernels import ops

    gen = torch.Generator().manual_seed(Hq * 100 + d)
    n, window, keep, scale = 300, 37, 11, 0.3
    keys, values = torch.randn((n, Hk, d), generator=gen), torch.randn((n, Hv, dv), generator=gen)
    positions = [0, 5, 10, 11, 12, 36, 37, 38, 46, 47, 48, 49, 63, 64, 100, 128, 200, 255, 256, 299]
    queries = torch.randn((len(positions), Hq, d), generator=gen)
    for i, p in enumerate(positions):
        # the query of head h likes the keys at the four edges, whoever sees them
        edge = [j for j in (p - window + 1, p - window, keep - 1, keep) if 0 <= j <= p]
        for h in range(Hq):
            queries[i, h] = sum(keys[j, h // (Hq // Hk)] for j in edge) * (6.0 / (scale * d)) + 0.3 * queries[i, h]
    if dtype == torch.bfloat16:
        keys, values, queries = (t.to(dtype).float() for t in (keys, values, queries))
    want = torch.stack([_plain_attention(queries[i], keys, values, p, window, keep, scale, Hq // Hk) for i, p in enumerate(positions)])
    off = torch.stack([_plain_attention(queries[i], keys, values, p, window + 1, keep, scale, Hq // Hk) for i, p in enumerate(positions)])
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    assert (want - off).abs().max() > 20 * tol  # (the planted keys do decide)
    k_pages, v_pages, table = _paged(keys, values, page, 120, gen)
    kp, vp = k_pages.to(DEV, dtype), v_pages.to(DEV, dtype)
    bt = table.to(DEV).view(1, -1)
    q = queries.reshape(len(positions), Hq * d).to(DEV, dtype)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    seq = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    kw = dict(v_head_dim=dv, keep_first=keep, value_heads=Hv)
    alone = ops.attention_generic(q, Hq, Hk, d, kp, vp, seq, pos, bt, window, scale, **kw).float().cpu().view(len(positions), Hq, dv)
    assert (alone.double() - want).abs().max() < tol * max(1.0, float(want.abs().max())), (alone.double() - want).abs().max()
    split = ops.attention_generic_split(q, Hq, Hk, d, kp, vp, seq, pos, bt, window, scale, longest=window, **kw).float().cpu().view_as(alone)
    assert torch.equal(split, alone)
    # a portion of a prompt: 40 consecutive positions, queries repeated (at least 32 tokens take the tiles through LDS)
    for first in (0, 3, 30, 120, 260):
        ps = list(range(first, first + 40))
        qs = queries[torch.arange(40) % len(positions)].reshape(40, Hq * d).to(DEV, dtype)
        tiled = ops.attention_generic(qs, Hq, Hk, d, kp, vp, torch.zeros(40, dtype=torch.int32, device=DEV),
                                      torch.tensor(ps, dtype=torch.int32, device=DEV), bt, window, scale, **kw).cpu()
        for i in (0, 7, 8, 9, 20, 39):
            one = ops.attention_generic(qs[i : i + 1], Hq, Hk, d, kp, vp, seq[:1], torch.tensor(ps[i : i + 1], dtype=torch.int32, device=DEV),
                                        bt, window, scale, **kw).cpu()
            assert torch.equal(tiled[i : i + 1], one), (first, i)
            ref = _plain_attention(qs[i].float().cpu().view(Hq, d), keys, values, ps[i], window, keep, scale, Hq // Hk)
            assert (one.float().view(Hq, dv).double() - ref).abs().max() < tol * max(1.0, float(ref.abs().max()))


@pytest.mark.parametrize("Hq,Hk,Hv,d,dv,page,window,keep", [
    (8, 2, 2, 128, 128, 16, 200, 20), (4, 4, 2, 64, 128, 16, 70, 64), (8, 4, 2, 128, 256, 32, 136, 70), (2, 2, 1, 32, 96, 16, 33, 5),
    (16, 1, 1, 64, 64, 8, 1000, 3), (4, 2, 1, 256, 256, 16, 100, 100), (6, 2, 2, 128, 128, 16, 64, 0)])
def test_matrix_core_attention_with_kept_first_keys_and_wide_values(Hq, Hk, Hv, d, dv, page, window, keep):
    """The split-KV decode kernel and the tiled prefill kernel against the plain kernel (which the test above holds
    against the formulas): a window that keeps first positions, values with fewer heads than the keys and rows that
    are a multiple of the keys' head size (worked off in calls of one head size each); queries that like the keys at
    the window's edges and at the end of the kept positions; single tokens at many positions, and portions of a
    prompt that begin before, at and behind the window's first full reach, behind a prefix in the cache."""
    from torchllms_amd.kernels import ops

    gen = torch.Generator().manual_seed(Hq + d + window)
    n, scale = 700, 0.7 / d ** 0.5
    keys = torch.randn((n, Hk, d), generator=gen).to(torch.bfloat16)
    values = torch.randn((n, Hv, dv), generator=gen).to(torch.bfloat16)
    k_pages, v_pages, table = _paged(keys.float(), values.float(), page, 2 * (n // page) + 9, gen)
    kp, vp = k_pages.to(DEV, torch.bfloat16), v_pages.to(DEV, torch.bfloat16)
    bt = table.to(DEV).view(1, -1)

    def queries_for(positions):
        q = torch.randn((len(positions), Hq, d), generator=gen)
        for i, p in enumerate(positions):
            edge = [j for j in (p - window + 1, p - window, keep - 1, keep) if 0 <= j <= p]
            for h in range(Hq):
                q[i, h] = sum(keys[j, h // (Hq // Hk)].float() for j in edge) * (5.0 / (scale * d)) + q[i, h]
        return q.reshape(len(positions), Hq * d).to(DEV, torch.bfloat16)

    kw = dict(keep_first=keep, value_heads=Hv)
    # single tokens
    positions = [0, 1, 15, 16, keep, keep + 1, window - 1, window, window + 1, window + keep - 1, window + keep, window + keep + 17, 300, 511, 512, 699]
    positions = sorted({min(max(p, 0), n - 1) for p in positions})
    q = queries_for(positions)
    pos = torch.tensor(positions, dtype=torch.int32, device=DEV)
    seq = torch.zeros(len(positions), dtype=torch.int32, device=DEV)
    want = ops.attention_generic(q, Hq, Hk, d, kp, vp, seq, pos, bt, window, scale, v_head_dim=dv, **kw).float()
    for split in (None, 64, 128):
        got = torch.zeros((len(positions), Hq * dv), dtype=torch.bfloat16, device=DEV)
        for at in range(0, dv, d):
            ops.attention_decode(q, Hq, Hk, d, kp, vp, seq, pos, bt, window, scale, min(max(positions) + 1, window + 15), out=got,
                                 split_size=split, v_offset=at, **kw)
        assert (got.float() - want).abs().max() < 3e-2 * max(1.0, float(want.abs().max())), (split, (got.float() - want).abs().max())
    # portions of a prompt behind what the cache holds already
    if not ops.prefill_attention_supported(torch.bfloat16, Hq, Hk, d, page):
        return
    qpt = ops.prefill_queries_per_tile(Hq, Hk, d)
    for first, count in ((0, 700), (0, 40), (keep + 3, 90), (window - 5, 130), (window + keep - 20, 77), (500, 200), (690, 10)):
        if first + count > n:  # (only what the cache holds)
            continue
        ps = list(range(first, first + count))
        q = queries_for(ps)
        qo = torch.tensor([0, count], dtype=torch.int32, device=DEV)
        kv = torch.tensor([first + count], dtype=torch.int32, device=DEV)
        rows, q0s = ops.prefill_tiles([0, count], 0, 1, qpt, [first + count], window)
        tiles = torch.tensor([rows, q0s], dtype=torch.int32, device=DEV)
        want = ops.attention_generic(q, Hq, Hk, d, kp, vp, torch.zeros(count, dtype=torch.int32, device=DEV),
                                     torch.tensor(ps, dtype=torch.int32, device=DEV), bt, window, scale, v_head_dim=dv, **kw).float()
        for groups in (1, 2):
            got = torch.zeros((count, Hq * dv), dtype=torch.bfloat16, device=DEV)
            for at in range(0, dv, d):
                ops.attention_prefill(q, Hq, Hk, d, kp, vp, qo, kv, bt, tiles[0], tiles[1], window, scale, got, key_groups=groups, v_offset=at, **kw)
            err = (got.float() - want).abs().max(dim=1).values
            assert float(err.max()) < 3e-2 * max(1.0, float(want.abs().max())), (first, count, groups, int(err.argmax()) + first, float(err.max()))


@pytest.mark.parametrize("S,D,n", [(3, 192, 70), (1, 64, 5), (4, 50, 33), (8, 36, 2), (16, 128, 9), (11, 30, 40)])
def test_streams_kernel_against_the_formulas(S, D, n):
    from torchllms_amd.kernels import ops

    gen = torch.Generator().manual_seed(S + D)
    x = torch.randn((S, n, D), generator=gen)
    y = torch.randn((n, D), generator=gen)
    mix, out_w, in_w = torch.randn((S, S), generator=gen), torch.randn(S, generator=gen), torch.randn(S, generator=gen)
    alpha, w, b = torch.tensor([0.7]), torch.randn(D, generator=gen), torch.randn(D, generator=gen)
    new = torch.einsum("sr,snd->rnd", mix.double(), x.double()) + out_w.double()[:, None, None] * y.double()[None]
    norm = lambda u: torch.tanh(0.7 * u) * w.double() + b.double()  # noqa: E731
    for dtype, tol in ((torch.float32, 2e-6), (torch.bfloat16, 1e-2)):
        xs = x.to(DEV).clone()
        rows = ops.streams_update(xs, branch=y.to(DEV, dtype), mix=mix.to(DEV), out_weights=out_w.to(DEV), read_weights=in_w.to(DEV),
                                  alpha=alpha.to(DEV), weight=w.to(DEV), bias=b.to(DEV), out_dtype=dtype)
        y_seen = y.to(dtype).double()
        new_seen = torch.einsum("sr,snd->rnd", mix.double(), x.double()) + out_w.double()[:, None, None] * y_seen[None]
        assert (xs.cpu().double() - new_seen).abs().max() < 1e-5
        want = norm(torch.einsum("s,snd->nd", in_w.double(), new_seen))
        assert rows.dtype == dtype and (rows.cpu().double() - want).abs().max() < tol * max(1.0, float(want.abs().max()))
    # the write alone, then the read alone give the same as both in one trip; a gathered read takes the plain sum
    xs = x.to(DEV).clone()
    ops.streams_update(xs, branch=y.to(DEV), mix=mix.to(DEV), out_weights=out_w.to(DEV))
    assert (xs.cpu().double() - new).abs().max() < 1e-5
    pick = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    got = ops.streams_update(xs, alpha=alpha.to(DEV), weight=w.to(DEV), bias=b.to(DEV), rows=pick, out_dtype=torch.float32)
    assert (got.cpu().double() - norm(new.sum(0))[[n - 1, 0]]).abs().max() < 1e-5
    opened = ops.streams_open(y.to(DEV), S)
    assert opened.shape == (S, n, D) and all(torch.equal(opened[s].cpu(), y) for s in range(S))


@pytest.mark.parametrize("H,dv", [(4, 96), (1, 7), (3, 256)])
def test_join_of_the_two_maps(H, dv):
    from torchllms_amd.kernels import ops

    gen = torch.Generator().manual_seed(dv)
    maps = torch.randn((19, 2, H, dv), generator=gen)
    lam, eps, gain = 0.37, 1e-5, 0.4
    o = maps[:, 0].double() - lam * maps[:, 1].double()
    want = (o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * gain).reshape(19, H * dv)
    got = ops.maps_join(maps.reshape(19, -1).to(DEV), H, dv, lam, eps, gain).cpu()
    assert (got.double() - want).abs().max() < 1e-5
    low = ops.maps_join(maps.reshape(19, -1).to(DEV, torch.bfloat16), H, dv, lam, eps, gain).float().cpu()
    assert (low.double() - want).abs().max() < 3e-2


def test_router_with_groups_against_the_plain_choice():
    """Scores drawn so that the best expert of a group that is shut out beats experts that are chosen; ties inside
    the score vector go to the lower index as ``topk`` of the plain function does for the drawn numbers."""
    from torchllms_amd.kernels import ops

    gen = torch.Generator().manual_seed(3)
    for E, count, keep, top, scale in ((10, 2, 1, 3, 1.5), (12, 4, 2, 5, 0.5), (6, 6, 3, 2, 1.0), (9, 1, 1, 4, 1.5), (64, 8, 3, 6, 1.0), (5, 0, 0, 2, 3.0)):
        z = torch.randn((200, E), generator=gen) * 2
        router = {"experts": E, "top": top, "scale": scale}
        if count:
            router["groups"] = {"count": count, "keep": keep}
        ids, weights = plain.routed_choice(z.double(), router)
        got_ids, got_w = ops.router_topk(z.to(DEV), E, None, top, groups=count, keep_groups=keep, normalize=True, scale=scale)
        assert torch.equal(got_ids.cpu().long(), ids), (E, count, keep, top)
        assert (got_w.cpu().double() - weights).abs().max() < 1e-6 * scale
        s = torch.softmax(z.double(), -1)
        assert (s.max(-1).indices != ids[:, 0]).sum() == 0  # the best expert's group always stays ...
        if count and keep < count and E // count > 1 and top > 1:  # ... and groups that close shut experts out that would have been chosen
            assert any(s[t].topk(top).indices.tolist() != ids[t].tolist() for t in range(200)), (E, count, keep, top)


def _plain_linear_attention(q, k, v, pre, bias, power, gate, norm_w, eps):
    n, H, dk = q.shape
    alpha = torch.sigmoid(pre.double().reshape(n, H, dk) + bias.double().reshape(H, dk)).pow(power)
    S = torch.zeros(H, dk, v.shape[-1], dtype=torch.float64)
    out = []
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t].double()[:, :, None] * v[t].double()[:, None, :]
        out.append(torch.einsum("hkv,hk->hv", S, q[t].double() * dk ** -0.5))
    o = torch.stack(out)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * norm_w.double()
    g = gate.double().reshape(n, H, -1)
    return (o * g * torch.sigmoid(g)).reshape(n, -1)


@pytest.mark.parametrize("H,dk,dv", [(4, 16, 24), (1, 200, 33), (3, 7, 5), (2, 128, 64)])
def test_gated_linear_attention_kernel(H, dk, dv):
    """Channels that forget at once beside channels that keep for hundreds of tokens, so that a decay applied to the
    wrong row, or one decay for a whole head, shows; a key written early and asked for late; one row, steps of a
    request through one slot, rows of several requests."""
    from torchllms_amd.kernels import ops

    n, eps, power = 300, 1e-5, 1.0 / 7.0
    gen = torch.Generator().manual_seed(dk + 2)
    qkv = torch.randn((n, 2 * H * dk + H * dv), generator=gen)
    pre = torch.randn((n, H * dk), generator=gen) * 2
    pre.reshape(n, H, dk)[:, :, ::3] += 12.0   # every third channel hardly decays
    pre.reshape(n, H, dk)[:, :, 1::3] -= 9.0   # its neighbour forgets within a few tokens
    gate = torch.randn((n, H * dv), generator=gen)
    qkv[5, H * dk : H * dk + dk : 3] *= 6.0     # a key that stands out in the channels that keep ...
    qkv[280, :dk] = qkv[5, H * dk : H * dk + dk]  # ... and a query that asks for it much later
    bias, norm_w = torch.randn(H * dk, generator=gen) * 0.5, torch.rand(dv, generator=gen) + 0.5
    q, k, v = qkv[:, : H * dk].reshape(n, H, dk), qkv[:, H * dk : 2 * H * dk].reshape(n, H, dk), qkv[:, 2 * H * dk :].reshape(n, H, dv)
    want = _plain_linear_attention(q, k, v, pre, bias, power, gate, norm_w, eps)
    x, pre_d, gate_d = qkv.to(DEV), pre.to(DEV), gate.to(DEV)
    consts = (bias.to(DEV), power)
    state = torch.zeros((3, H * dv * dk + 4), device=DEV)
    rows = torch.tensor([0, n], dtype=torch.int32, device=DEV)
    slot0 = torch.tensor([0], dtype=torch.int32, device=DEV)
    whole = ops.gated_linear(x, pre_d, *consts, gate_d, 0, norm_w.to(DEV), eps, state, 4, rows, slot0, H, dk, dv).cpu()
    assert (whole.double() - want).abs().max() < 3e-4 * want.abs().max(), (whole.double() - want).abs().max()
    assert float(state[0, :4].abs().max()) == 0.0 and float(state[1].abs().max()) == 0.0
    state2 = torch.zeros_like(state)
    slot1 = torch.tensor([1], dtype=torch.int32, device=DEV)
    out, at = [], 0
    for m in [1, 1, 15, 16, 17, 2, 1, 33, 1, 64, 1, 1, 100, 1, 5, 1, 40]:
        out.append(ops.gated_linear(x[at : at + m].contiguous(), pre_d[at : at + m].contiguous(), *consts, gate_d[at : at + m].contiguous(), 0,
                                    norm_w.to(DEV), eps, state2, 4, torch.tensor([0, m], dtype=torch.int32, device=DEV), slot1, H, dk, dv).cpu())
        at += m
    assert at == n
    assert torch.equal(torch.cat(out), whole)
    assert torch.equal(state2[1], state[0])
    # rows of one step that belong to different requests: each starts from its own (zero) state
    rows3 = torch.tensor([0, 100, 101, n], dtype=torch.int32, device=DEV)
    batch = ops.gated_linear(x, pre_d, *consts, gate_d, 0, norm_w.to(DEV), eps, torch.zeros_like(state), 4, rows3,
                             torch.arange(3, dtype=torch.int32, device=DEV), H, dk, dv).cpu()
    assert torch.equal(batch[:100], whole[:100])
    want3 = _plain_linear_attention(q[101:], k[101:], v[101:], pre[101:], bias, power, gate[101:], norm_w, eps)
    assert (batch[101:].double() - want3).abs().max() < 3e-4 * want3.abs().max()
    # what lies far back matters: without the first hundred tokens the late rows are others
    assert (want3[150:] - want[251:]).abs().max() > 1e-2 * want.abs().max()


# ----------------------------------------------------------------------------- far keys, edges, slots, long decoding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_with_sharp_attention_and_long_memory(tmp_path, dtype):
    """Scores with a spread of four make every query look at a few keys anywhere in its window of some hundred
    positions and among the kept first ones, decays near one keep what the first tokens wrote: a lost page, a key one
    off, a kept page given back or a state that was not carried shows in the logits of late positions; whole, in
    portions that end at and beside page borders and window edges, and decoded one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = models.model(97, 64, 3, 2.0, 1e-5, [
        # (heads of 32 channels with values twice as wide: in bfloat16 the matrix-core kernels run them, the reader below too)
        models.layer("attention", models.diff_attention(2, 1, 32, 64, 0.2, 0.5, _R(32, 1e5), 300, keep_first=17, conv=3), models.moe(32, 4, 2, 2.0, groups=(2, 1), shared=16)),
        models.layer("parallel", models.pair(models.left(4, 2, 32, 32, 0.2, _R(16, 1e4, (4.0, 128, 16.0, 1.0)), 130, keep_first=40),
                                             models.right(2, 32, 32, 64.0, 8), 1.0, 0.6), None),
        models.layer("attention", models.diff_attention(4, 1, 32, 64, 0.2, 0.3, _R(32, 1e5), 129, keep_first=33, conv=2, kv_from=0), None),
        models.layer("latent_attention", models.latent(2, 32, 16, 32, 48, 0.15, 257, scaling=(2.0, 256, 32.0, 1.0)), models.moe(24, 3, 1, 1.0)),
    ])
    folder = folder_for(dtype, tmp_path / "m", cfg_dict, seed=3, sharpen=4.0)
    cfg, weights = models.read_folder(folder)
    tokens = random_tokens(700, cfg["vocab"], 5)
    truth, scale = truth_of(cfg, weights, {"r": tokens})
    page = 16
    engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=2 * 45, max_seqs=2)
    tol = FP32_TOL if dtype == "float32" else BF16_TOL
    engine.admit("w")
    whole = engine.step([StepEntry("w", tokens, list(range(700)))]).cpu()
    engine.free("w")
    engine.admit("c")
    rows, at = [], 0
    for n in [16, 15, 1, 2, 30, 33, 31, 64, 63, 1, 129, 127, 2, 100] + [1] * 86:
        rows.append(engine.step([StepEntry("c", tokens[at : at + n], list(range(n)))]).cpu())
        at += n
        engine.cache.check_invariants()
    assert at == 700
    # the windows have passed most of the prompt: its pages are back but for those of the kept first positions
    assert all(engine.cache.block_table("c", g)[0] >= 0 for g, spec in enumerate(engine.cache.groups) if spec.keep_first)
    assert any(-1 in engine.cache.block_table("c", g) for g in range(len(engine.cache.groups)))
    cut = torch.cat(rows)
    for name, got in (("whole", whole), ("cut", cut)):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(700)]
        if dtype == "float32":
            assert max(dists) < tol, f"{name}: distance {max(dists)} at {dists.index(max(dists))}"
        else:
            assert_within_rounding(dists, tol, name)
    if dtype == "float32":
        assert torch.equal(whole, cut)
    # dropping what lies far back would be seen: the truth of the last 100 tokens alone is another
    short = plain.forward(cfg, weights, tokens[600:])
    if dtype == "float32":  # (the sharp comparison is the one that sees it)
        assert max(distance(short[i], truth["r"][600 + i], scale) for i in range(50, 100)) > 100 * tol


def test_a_slot_that_is_used_again_starts_from_zero(tmp_path):
    """One state slot and few pages: each request takes over what the one before left (the linear attention's state,
    the convolutions' histories, pages of keys, kept first pages), and must not see any of it."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=8)
    cfg, weights = models.read_folder(folder)
    requests = {f"q{i}": random_tokens(n, cfg["vocab"], 30 + i) for i, n in enumerate([50, 3, 64, 20])}
    truth, scale = truth_of(cfg, weights, requests)
    engine = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=8, max_seqs=1)
    for rid, toks in requests.items():
        engine.admit(rid)
        head = max(len(toks) - 5, 1)
        rows = [engine.step([StepEntry(rid, toks[:head], list(range(head)))]).cpu()]
        rows += [engine.step([StepEntry(rid, [t], [0])]).cpu() for t in toks[head:]]
        engine.free(rid)
        got = torch.cat(rows)
        assert max(distance(got[i], truth[rid][i], scale) for i in range(len(toks))) < FP32_TOL, rid
    engine.cache.check_invariants()


def test_long_decoding_from_recorded_steps(tmp_path):
    """Three requests decode 150 tokens together, over window edges and kept first positions: the steps are replayed
    from HIP graphs after the first few, states and histories move on with every replay, pages behind the windows go
    back while the kept ones stay, and the logits stay the plain model's."""
    from torchllms_amd.engine import Engine, StepEntry

    requests = {f"d{i}": random_tokens(170 + 7 * i, models.CONFIG_B["vocab"], 60 + i) for i in range(3)}
    for dtype, tol in (("float32", FP32_TOL), ("bfloat16", BF16_TOL)):
        folder = folder_for(dtype, tmp_path / "m", models.CONFIG_B, seed=12)
        truth, scale = truth_of(*models.read_folder(folder), requests)
        engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=40, max_seqs=3)
        for rid in requests:
            engine.admit(rid)
        engine.step([StepEntry(rid, toks[: len(toks) - 150], []) for rid, toks in requests.items()])
        dists = []
        for j in range(150):
            entries = [StepEntry(rid, [toks[len(toks) - 150 + j]], [0]) for rid, toks in requests.items()]
            logits = engine.step(entries).cpu()
            for row, (rid, toks) in zip(logits, requests.items()):
                dists.append(distance(row, truth[rid][len(toks) - 150 + j], scale))
        engine.cache.check_invariants()
        if dtype == "float32":
            assert max(dists) < tol, f"{dtype}: {max(dists)}"
        else:
            assert_within_rounding(dists, tol, dtype)
        assert engine.graphs is not None and any(g.replays > 100 for g in engine.graphs.graphs.values())


# ----------------------------------------------------------------------------- through the entry point
def test_greedy_generation_through_the_entry_point(tmp_path):
    """``LLM.generate``: the scheduler admits, cuts prompts into portions under a small token budget, decodes
    everybody together and frees; the tokens are the plain model's."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=4)
    cfg, weights = models.read_folder(folder)
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (5, 37, 1, 64, 22)]
    new = 20

    def plain_greedy(prompt):
        toks = list(prompt)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, weights, toks)[-1].argmax()))
        return toks[len(prompt):]

    llm = LLM(str(folder), precision="float32", max_len=128, max_bsz=3, page_size=8, max_num_batched_tokens=24)
    results = llm.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=new)
    for p, r in zip(prompts, results):
        assert r.token_ids == plain_greedy(p)
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []
    llm16 = LLM(str(folder), precision="bfloat16", max_len=128, max_bsz=3, page_size=8)
    for p, r in zip(prompts, llm16.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=4)):
        logits = plain.forward(cfg, weights, p)[-1]
        assert logits[r.token_ids[0]] >= logits.max() - 0.05 * float(logits.std())


def test_a_preempted_request_starts_again_from_clean_state(tmp_path):
    """Too few pages for four requests: the scheduler takes the youngest off, gives its pages and its slot away and
    later computes it again from its prompt and what it had generated; the sampled tokens are those of the run with
    room for everybody."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIG_B, seed=9)
    cfg, _ = models.read_folder(folder)
    prompts = [random_tokens(n, cfg["vocab"], 80 + n) for n in (30, 25, 28, 21)]
    ample = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8)
    want = ample.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    tight = LLM(str(folder), precision="float32", max_len=96, max_bsz=4, page_size=8, num_pages=20)
    got = tight.generate(prompt_token_ids=prompts, temperature=0.8, max_new_tokens=30, seed=7)
    assert tight.last_stats["preemptions"] > 0
    assert [r.token_ids for r in got] == [r.token_ids for r in want]
    tight.engine.cache.check_invariants()


def test_generate_command_line_with_random_weights(tmp_path):
    """The generate program given nothing but a config.json: ``--random-weights --seed`` draws the weights that
    ``write_model_folder`` would write for that seed, so the plain model can say which tokens to expect."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    from torchllms_amd.config.nosuzen import NosuzenConfig
    from torchllms_amd.weights import write_model_folder

    root = Path(__file__).resolve().parent.parent
    folder = tmp_path / "only_config"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(models.CONFIG_B))
    prompt = random_tokens(13, models.CONFIG_B["vocab"], 21)
    proc = subprocess.run(
        [sys.executable, "-m", "torchllms_amd.inference.generate", "--model", str(folder), "--dtype", "float32", "--random-weights",
         "--seed", "7", "--max-new-tokens", "6", "--prompt-ids", *map(str, prompt)],
        capture_output=True, text=True, cwd=root, timeout=300,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.split()[-6:]]
    written = write_model_folder(tmp_path / "written", NosuzenConfig.from_dict(models.CONFIG_B), seed=7, dtype=torch.float32)
    cfg, weights = models.read_folder(written)
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(plain.forward(cfg, weights, toks)[-1].argmax()))
    assert got == toks[len(prompt):]


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a user starts it: steps on standard input, logits files out, a pool for the live tokens
    only, four slots."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    folder = models.make_folder(tmp_path / "m", models.CONFIG_C, seed=6)
    cfg, weights = models.read_folder(folder)
    requests = {f"t{i}": random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate([80, 33, 120, 64, 50, 90])}
    truth, scale = truth_of(cfg, weights, requests)
    steps = schedules.mixed(requests)
    out = tmp_path / "out"
    prog = Path(__file__).resolve().parents[1] / "bin" / "trace_run"
    run = subprocess.run([sys.executable, str(prog), "--model", str(folder), "--dtype", "float32", "--out", str(out), "--max-tokens",
                          str(schedules.max_live_tokens(steps))], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=600)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [ln for ln in run.stdout.splitlines() if ln.startswith("done")] == [f"done {s['step']}" for s in steps]
    for s, where in zip(steps, schedules.positions_of(steps)):
        if not where:
            continue
        got = torch.from_numpy(np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(len(where), cfg["vocab"]))
        for (rid, pos), row in zip(where, got):
            assert distance(row, truth[rid][pos], scale) < FP32_TOL, (s["step"], rid, pos)


ODD = {
    "width_50": models.model(33, 50, 3, 1.5, 1e-5, [
        models.layer("attention", models.diff_attention(3, 1, 10, 6, 0.3, 0.5, _R(6, 100.0), 9, keep_first=2, conv=2), models.moe(14, 3, 2, 1.5, shared=10)),
        models.layer("parallel", models.pair(models.left(2, 1, 12, 10, 0.3, _R(4, 100.0), 7, keep_first=1), models.right(2, 6, 10, 3.0, 2), 0.8, 0.7), None),
        models.layer("latent_attention", models.latent(3, 6, 2, 10, 14, 0.3, 11), models.moe(9, 2, 1, 1.0, groups=(2, 1))),
        models.layer("attention", models.diff_attention(1, 1, 10, 6, 0.3, 0.2, _R(6, 100.0), 30, keep_first=0, kv_from=0), None),
    ]),
    "width_52": models.model(70, 52, 5, 1.0, 1e-5, [
        models.layer("latent_attention", models.latent(1, 4, 4, 4, 12, 0.4, 1000), models.moe(12, 4, 2, 2.0, groups=(2, 2), shared=20)),
        models.layer("attention", models.diff_attention(2, 2, 4, 12, 0.4, 0.9, _R(4, 10.0), 5, keep_first=5, conv=3), None),
    ]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD))
def test_widths_that_are_no_multiple_of_eight(tmp_path, name, dtype):
    """Rows that no 16-byte load fits, heads of a handful of channels, more streams than usual: the kernels' plain forms."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = folder_for(dtype, tmp_path / name, ODD[name], seed=2)
    cfg, weights = models.read_folder(folder)
    tokens = random_tokens(90, cfg["vocab"], 4)
    truth, scale = truth_of(cfg, weights, {"r": tokens})
    engine = Engine.from_folder(folder, dtype=dtype, page_size=4, num_pages=60, max_seqs=2)
    engine.admit("whole")
    whole = engine.step([StepEntry("whole", tokens, list(range(90)))]).cpu()
    engine.admit("cut")
    rows, at = [], 0
    for n in (3, 2, 40, 1, 1, 35, 1, 1, 1, 5):
        rows.append(engine.step([StepEntry("cut", tokens[at : at + n], list(range(n)))]).cpu())
        at += n
    assert at == 90
    cut = torch.cat(rows)
    for what, got in (("whole", whole), ("cut", cut)):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(90)]
        if dtype == "float32":
            assert max(dists) < FP32_TOL, f"{name}/{what}: {max(dists)}"
        else:
            assert_within_rounding(dists, 2 * BF16_TOL, f"{name}/{what}")
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- random configurations
def random_config(seed: int) -> dict:
    """A Nosuzen configuration drawn from a seed: every size, constant and the order of layers."""
    import random

    rng = random.Random(seed)
    width = rng.choice([40, 64, 72, 96, 128, 160])

    def rotation(most):
        dims = rng.choice([0, most // 2, most]) // 2 * 2
        scaling = rng.choice([None, (rng.choice([2.0, 4.0, 16.0]), rng.choice([16, 64, 256]), rng.choice([4.0, 32.0]), rng.choice([1.0, 2.0]))])
        return _R(dims, rng.choice([100.0, 10000.0, 1000000.0]), scaling)

    layers, owners = [], []
    for i in range(rng.randint(2, 6)):
        experts = rng.choice([1, 2, 4, 6, 9, 12])
        count = rng.choice([None] + [c for c in (1, 2, 3, 4, 6) if experts % c == 0])
        keep = rng.randint(1, count) if count else None
        top = rng.randint(1, (keep * (experts // count)) if count else experts)
        mlp = rng.choice([None, models.moe(rng.choice([16, 24, 40, 72]), experts, top, rng.choice([0.5, 1.0, 2.5]),
                                           groups=(count, keep) if count else None, shared=rng.choice([None, 16, 56]))])
        kind = rng.choice(["attention", "attention", "latent_attention", "parallel"])
        size, keep_first = rng.choice([1, 7, 16, 33, 64, 129, 1000]), rng.choice([0, 0, 1, 5, 16, 40])
        if kind == "attention":
            if owners and rng.random() < 0.5:
                src = rng.choice(owners)
                m = dict(layers[src]["mixer"])
                m.update(kv_from=src, heads=m["kv_heads"] * rng.choice([1, 2, 4]), diff=rng.choice([0.1, 0.5, 0.8]), rot=dict(m["rot"]),
                         mask={"size": size, "keep_first": keep_first})
                if rng.random() < 0.5:
                    m["conv"] = rng.choice([1, 2, 4])
            else:
                kv = rng.choice([1, 2, 3])
                dim = rng.choice([8, 16, 24, 48, 64])
                m = models.diff_attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([8, 16, 40, 96, 128]), rng.choice([0.1, 0.3, 1.0]) * 16 / dim,
                                          rng.choice([0.1, 0.5, 0.8]), rotation(dim), size, keep_first, conv=rng.choice([None, 1, 2, 3, 4]))
                owners.append(i)
            layers.append(models.layer("attention", m, mlp))
        elif kind == "latent_attention":
            rot_dim = rng.choice([0, 8, 16, 32])
            rt = rotation(rot_dim)
            rt["dims"] = rot_dim
            m = models.latent(rng.choice([1, 2, 3, 4]), rng.choice([8, 16, 32]), rot_dim, rng.choice([8, 16, 40]), rng.choice([24, 48, 96, 112, 224]),
                              rng.choice([0.1, 0.2]), size)
            m["rot"] = rt
            layers.append(models.layer("latent_attention", m, mlp))
        else:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([16, 24, 32, 64, 128])
            lf = models.left(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([dim, dim, 8, 40]), rng.choice([0.1, 0.3, 1.0]) * 16 / dim, rotation(dim), size, keep_first)
            rt = models.right(rng.choice([1, 2, 3]), rng.choice([8, 20, 32, 64, 128, 192]), rng.choice([8, 24, 32, 64, 100]), rng.choice([1.0, 4.0, 16.0, 64.0]),
                              rng.choice([1, 4, 16, 24]))
            layers.append(models.layer("parallel", models.pair(lf, rt, rng.choice([0.3, 0.6, 1.0]), rng.choice([0.5, 1.0, 1.4])), mlp))
    return models.model(rng.choice([50, 97, 256, 301]), width, rng.choice([1, 2, 3, 4, 5]), rng.choice([1.0, 0.5, 12.0]), rng.choice([1e-5, 1e-6, 1e-3]), layers)


@pytest.mark.parametrize("seed", range(10))
def test_random_configurations(tmp_path, seed):
    """Sizes nobody chose: a prompt whole, and the same tokens in portions, single tokens and beside a second
    request, in both dtypes, against the plain model."""
    import random

    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = random_config(3000 + seed)
    rng = random.Random(seed)
    requests = {"a": random_tokens(rng.randint(120, 330), cfg_dict["vocab"], seed), "b": random_tokens(rng.randint(20, 90), cfg_dict["vocab"], seed + 50)}
    page = rng.choice([4, 8, 16, 32])
    # (drawn constants can put a head's two maps close to cancelling, where the join magnifies 32-bit rounding several
    # times, in the plain model run in 32-bit as well; a wrong key, mask or state is a hundred times the bound)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 2 * BF16_TOL)):
        folder = folder_for(dtype, tmp_path / "m", cfg_dict, seed=seed)
        truth, scale = truth_of(*models.read_folder(folder), requests)
        seen = []
        engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=2 * (-(-420 // page)) + 4, max_seqs=3)
        engine.admit("w")
        whole = engine.step([StepEntry("w", requests["a"], list(range(len(requests["a"]))))]).cpu()
        engine.free("w")
        for i, row in enumerate(whole):
            d = distance(row, truth["a"][i], scale)
            seen.append(d)
            assert dtype == "bfloat16" or d < tol, f"{dtype} whole at {i}: {d}  {cfg_dict}"
        at = {"a": 0, "b": 0}
        engine.admit("a")
        engine.admit("b")
        while at["a"] < len(requests["a"]) or at["b"] < len(requests["b"]):
            entries = []
            for rid in ("a", "b"):
                left = len(requests[rid]) - at[rid]
                if left and rng.random() < 0.8:
                    n = min(left, rng.choice([1, 1, 2, 3, 17, 40, 64, 130]))
                    entries.append(StepEntry(rid, requests[rid][at[rid] : at[rid] + n], list(range(n))))
            if not entries:
                continue
            logits = engine.step(entries).cpu()
            engine.cache.check_invariants()
            k = 0
            for e in entries:
                for w in e.want:
                    d = distance(logits[k], truth[e.rid][at[e.rid] + w], scale)
                    seen.append(d)
                    assert dtype == "bfloat16" or d < tol, f"{dtype} {e.rid} at {at[e.rid] + w} in a step of {[len(x.tokens) for x in entries]}: {d}  {cfg_dict}"
                    if dtype == "float32" and e.rid == "a":
                        assert torch.equal(logits[k], whole[at["a"] + w])
                    k += 1
                at[e.rid] += len(e.tokens)
        if dtype == "bfloat16":
            assert_within_rounding(seen, tol, f"{cfg_dict}")
        del engine
