"""The Kepevik decoder in the engine against the plain implementation of tests/plain/kepevik.py: every mechanism
alone, whole prompts against decoding token by token, portions down to two tokens, mixed batches with pages and
state slots that are used again, keys and written tokens far back, long decoding from recorded graphs, and greedy
generation through ``LLM.generate`` and the scheduler; on three small configurations that differ in every size, in
32-bit and in bfloat16.  The kernels that are new with this design are also compared alone, on inputs made so that
every branch of theirs is taken."""

import math

import pytest
import torch

from . import kepevik_models as models
from . import schedules
from .helpers import random_tokens
from .plain import kepevik as plain
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [70, 41, 100, 35, 50, 33], "B": [66, 40, 130, 35, 90], "C": [45, 150, 37, 64, 120]}
#: distances are measured as a replay of a trace is judged: the difference of two rows of logits with its mean taken
#: off, root mean square over the vocabulary, over the root mean square of the truth
FP32_TOL = 3e-5
BF16_TOL = 5e-2


def distance(got: torch.Tensor, truth: torch.Tensor, scale: float) -> float:
    d = got.double() - truth.double()
    d = d - d.mean()
    return float(d.pow(2).mean().sqrt()) / scale


def truth_of(cfg, weights, requests):
    w64 = {k: v.double() for k, v in weights.items()}
    out = {rid: plain.forward(cfg, w64, toks) for rid, toks in requests.items()}
    scale = float(torch.cat([(t - t.mean(-1, keepdim=True)).flatten() for t in out.values()]).pow(2).mean().sqrt())
    return out, scale


def folder_for(dtype, path, cfg_dict, **kw):
    """The model a run in ``dtype`` is compared on.  Rounding to bfloat16 moves a router's scores by a thousandth,
    and where two outputs lie closer than that the engine and the plain model choose different experts for a token:
    that position is then another model's output, and the positions behind it feel it through the states.  With
    corrections of the scores' own spread such calls are a few in a thousand, enough to spoil a comparison; so
    bfloat16 runs get routers whose corrections decide the choice, and the 32-bit runs, which are the sharp ones,
    get routers whose choice changes from token to token."""
    return models.make_folder(path / dtype, cfg_dict, decisive_router=dtype == "bfloat16", **kw)


def assert_within_rounding(dists, tol, what):
    """bfloat16 against the plain model: all but 3% of the positions lie under the bound, and their mean under half
    of it (four layers on a stream of 64 channels, with projections five times the usual size, reach 0.02 by
    rounding alone, the same in every schedule); a fault of a kernel moves every position."""
    d = sorted(dists)
    keep = d[: max(len(d) - max(len(d) * 3 // 100, 1), 1)]
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
    tmp = tmp_path_factory.mktemp("kepevik")
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
    """Every 32-bit kernel adds in an order fixed by the element it computes (the recurrences token by token, the
    experts pair by pair in the order of a token's choices), so cutting, batching, pages and slots change no bit."""
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
_TINY_LEFT = models.left(1, 1, 8, 0, 0.3)
_TINY_RIGHT = models.right(1, 1, 8, 8, 1, 4, 4)
_TINY_MEMORY = models.mlstm(1, 4, 4, 5.0)
ALONE = {
    "memory": models.layer("mlstm", models.mlstm(4, 24, 40, 12.0)),
    "memory_wide_keys": models.layer("mlstm", models.mlstm(1, 256, 31, 6.0)),
    "memory_odd": models.layer("mlstm", models.mlstm(3, 18, 70, 2.0)),
    "memory_one_value": models.layer("mlstm", models.mlstm(2, 64, 1, 30.0)),
    # one side of a parallel layer alone: the other's weight is zero
    "softmax_side": models.layer("parallel", models.pair(models.left(4, 2, 24, 10, 0.25), _TINY_RIGHT, 1.3, 0.0)),
    "softmax_side_matrix_cores_64": models.layer("parallel", models.pair(models.left(8, 2, 64, 32, 0.2), _TINY_RIGHT, 1.0, 0.0)),
    "softmax_side_matrix_cores_128": models.layer("parallel", models.pair(models.left(4, 1, 128, 128, 0.1, base=300.0), _TINY_RIGHT, 0.5, 0.0)),
    "delta_side": models.layer("parallel", models.pair(_TINY_LEFT, models.right(4, 2, 24, 40, 4, 6, 9), 0.0, 1.2)),
    "delta_side_wide": models.layer("parallel", models.pair(_TINY_LEFT, models.right(1, 1, 256, 64, 2, 32, 16), 0.0, 0.7)),
    "delta_side_odd": models.layer("parallel", models.pair(_TINY_LEFT, models.right(3, 1, 18, 70, 3, 3, 5), 0.0, 1.0)),
    "both_sides": models.layer("parallel", models.pair(models.left(2, 1, 32, 32, 0.2), models.right(2, 2, 32, 16, 5, 8, 8), 0.6, 0.5)),
    "dense": models.layer("mlstm", _TINY_MEMORY, models.dense(136)),
    "routed": models.layer("mlstm", _TINY_MEMORY, models.moe(40, 6, 3, identity=2, shared=56)),
    "routed_one_choice": models.layer("mlstm", _TINY_MEMORY, models.moe(33, 5, 1)),
    "routed_all_chosen": models.layer("mlstm", _TINY_MEMORY, models.moe(16, 2, 3, identity=1, shared=8)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("what", sorted(ALONE))
def test_a_mechanism_alone(tmp_path, what, dtype):
    """A model of one layer with that mixer and no feed-forward (or hardly a mixer and a feed-forward), a prompt in
    one step and, in a second request, the same tokens in portions and one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    folder = folder_for(dtype, tmp_path / what, models.single_layer(ALONE[what]), seed=5, sharpen=3.0)
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
    assert at == len(tokens)
    cut = torch.cat(rows)
    for name, got in (("whole", whole), ("cut", cut)):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(len(tokens))]
        if dtype == "float32":
            assert max(dists) < FP32_TOL, f"{what}/{name}: distance {max(dists)}"
        else:
            assert_within_rounding(dists, BF16_TOL, f"{what}/{name}")
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- the new kernels alone
def _rows(n_tokens, cuts, dev):
    """Row offsets of a step that holds ``n_tokens`` tokens cut into rows at ``cuts``, and a slot for each row."""
    bounds = [0] + list(cuts) + [n_tokens]
    return (torch.tensor(bounds, dtype=torch.int32, device=dev), torch.arange(len(bounds) - 1, dtype=torch.int32, device=dev))


def _plain_memory(proj, H, dk, dv, i_b, f_b, norm_w, cap, eps):
    """The plain cell on ready projections: the weights are slices of an identity, so h is the projection."""
    n, width = proj.shape
    eye = torch.eye(width, dtype=torch.float64)
    qk, v = H * dk, H * dv
    w = {"x.q": eye[:qk], "x.k": eye[qk : 2 * qk], "x.v": eye[2 * qk : 2 * qk + v], "x.g": eye[2 * qk + v : 2 * qk + 2 * v],
         "x.i": eye[2 * qk + 2 * v : 2 * qk + 2 * v + H], "x.f": eye[2 * qk + 2 * v + H :], "x.i.b": i_b.double(), "x.f.b": f_b.double(),
         "x.norm": norm_w.double(), "x.o": torch.eye(v, dtype=torch.float64)}
    return plain.matrix_memory(proj.double(), w, "x.", {"heads": H, "dim": dk, "vdim": dv, "gate_cap": cap}, eps)


@pytest.mark.parametrize("H,dk,dv", [(2, 16, 24), (1, 200, 33), (3, 7, 5), (2, 128, 64)])
def test_matrix_memory_kernel_on_gates_of_every_kind(H, dk, dv):
    """Input gates that jump far above the running maximum and fall far below it, forget gates that keep everything
    and that drop everything, gates beyond the cap, a normaliser that is smaller than its floor and one that is
    larger, a token whose written key stands out and is read back hundreds of tokens later; a sequence in one row,
    and the same cut into rows of a step that follow each other through the state."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    n, cap, eps = 330, 9.0, 1e-5
    g = torch.Generator().manual_seed(dk)
    qk, v = H * dk, H * dv
    proj = torch.randn((n, 2 * qk + 2 * v + 2 * H), generator=g)
    gi, gf = proj[:, 2 * qk + 2 * v : 2 * qk + 2 * v + H], proj[:, 2 * qk + 2 * v + H :]
    gi.mul_(3.0)
    gf.mul_(2.0).add_(3.0)
    gi[40] = 30.0       # beyond the cap, and far above every maximum so far
    gi[41:60] = -30.0   # then nothing is written for a while
    gf[100:104] = -40.0  # everything is dropped: the maximum falls, the floor exp(-m) rises above |n . q|
    gi[100:110] = -6.0
    gf[200:] += 6.0     # and a stretch that forgets almost nothing
    proj[7, qk : 2 * qk] *= 8.0  # a key that stands out ...
    proj[300, :qk] = proj[7, qk : 2 * qk] / 8.0  # ... and a query that asks for it much later
    i_b, f_b, norm_w = torch.randn(H, generator=g), torch.randn(H, generator=g), torch.rand(H * dv, generator=g) + 0.5
    want = _plain_memory(proj, H, dk, dv, i_b, f_b, norm_w, cap, eps)
    size = ops.matrix_memory_state_size(H, dk, dv)
    args = (0, qk, 2 * qk, 2 * qk + 2 * v, 2 * qk + 2 * v + H, 2 * qk + v, i_b.to(dev), f_b.to(dev), cap, norm_w.to(dev), eps)
    x = proj.to(dev)
    state = torch.zeros((3, size + 5), device=dev)
    rows, slots = _rows(n, [], dev)
    whole = ops.matrix_memory(x, *args, state, 5, rows, slots, H, dk, dv).cpu()
    assert (whole.double() - want).abs().max() < 2e-4 * want.abs().max(), (whole.double() - want).abs().max()
    assert float(state[0, :5].abs().max()) == 0.0 and float(state[1].abs().max()) == 0.0
    # the same tokens as steps of one request: portions of many sizes and single tokens, through slot 2
    state2 = torch.zeros_like(state)
    one_row = torch.tensor([2], dtype=torch.int32, device=dev)
    out, at = [], 0
    for m in [1, 1, 15, 16, 17, 2, 1, 33, 1, 64, 1, 1, 100, 1, 5, 1, 70]:
        out.append(ops.matrix_memory(x[at : at + m].contiguous(), *args, state2, 5, torch.tensor([0, m], dtype=torch.int32, device=dev),
                                     one_row, H, dk, dv).cpu())
        at += m
    assert at == n
    assert torch.equal(torch.cat(out), whole)
    assert torch.equal(state2[2], state[0])
    # and as rows of one step that belong to different requests: each starts from its own (zero) state
    rows3, slots3 = _rows(n, [100, 101], dev)
    state3 = torch.zeros_like(state)
    batch = ops.matrix_memory(x, *args, state3, 5, rows3, slots3, H, dk, dv).cpu()
    assert torch.equal(batch[:100], whole[:100])
    want3 = _plain_memory(proj[101:], H, dk, dv, i_b, f_b, norm_w, cap, eps)
    assert (batch[101:].double() - want3).abs().max() < 2e-4 * want3.abs().max()
    low = ops.matrix_memory(x.to(torch.bfloat16), *args, torch.zeros_like(state), 5, rows, slots, H, dk, dv).float().cpu()
    want16 = _plain_memory(proj.to(torch.bfloat16).float(), H, dk, dv, i_b, f_b, norm_w, cap, eps)
    assert (low.double() - want16).abs().max() < 2e-2 * want16.abs().max()


def _plain_delta(qkv, b, a, gate, H, G, dk, dv, A_log, dt_bias, norm_w, eps):
    """The plain delta rule on ready projections (one tap of convolution with weight one would add a silu, so the
    recurrence is restated here from the mixer's formulas; the mixer itself is compared through the engine)."""
    n = qkv.shape[0]
    q = qkv[:, : G * dk].reshape(n, G, dk).double()
    k = qkv[:, G * dk : 2 * G * dk].reshape(n, G, dk).double()
    v = qkv[:, 2 * G * dk :].reshape(n, H, dv).double()
    q = q / torch.sqrt((q ** 2).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k ** 2).sum(-1, keepdim=True) + 1e-6)
    beta = plain.sigmoid(b.double())
    decay = torch.exp(-torch.exp(A_log.double())[None, :, None] * plain.softplus(a.double().reshape(n, H, dk) + dt_bias.double().reshape(H, dk)))
    out = torch.zeros(n, H, dv, dtype=torch.float64)
    for h in range(H):
        gq = h // (H // G)
        M = torch.zeros(dk, dv, dtype=torch.float64)
        for t in range(n):
            M = decay[t, h][:, None] * M
            u = beta[t, h] * (v[t, h] - M.T @ k[t, gq])
            M = M + torch.outer(k[t, gq], u)
            out[t, h] = M.T @ q[t, gq]
    out = plain.rms_unit(out, eps) * norm_w.double()
    return (out * plain.sigmoid(gate.double().reshape(n, H, dv))).reshape(n, H * dv)


@pytest.mark.parametrize("H,G,dk,dv", [(4, 2, 16, 24), (1, 1, 200, 33), (3, 1, 7, 5), (2, 2, 128, 64)])
def test_delta_rule_with_a_decay_per_channel(H, G, dk, dv):
    """Channels that forget at once beside channels that keep for hundreds of tokens, so that a decay applied to the
    wrong row, or one decay for a whole head, shows; a key written early and asked for late; one row, steps of a
    request, rows of several requests."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    n, eps = 300, 1e-5
    g = torch.Generator().manual_seed(dk + 1)
    qkv = torch.randn((n, 2 * G * dk + H * dv), generator=g)
    b = torch.randn((n, H), generator=g) * 2
    a = torch.randn((n, H * dk), generator=g) * 2
    a.reshape(n, H, dk)[:, :, ::3] -= 12.0  # every third channel hardly decays
    a.reshape(n, H, dk)[:, :, 1::3] += 6.0  # its neighbour forgets within a token or two
    gate = torch.randn((n, H * dv), generator=g)
    qkv[5, G * dk : G * dk + dk : 3] *= 6.0
    qkv[280, :dk] = qkv[5, G * dk : G * dk + dk]
    A_log, dt_bias, norm_w = torch.randn(H, generator=g) * 0.5, torch.randn(H * dk, generator=g) * 0.5, torch.rand(dv, generator=g) + 0.5
    want = _plain_delta(qkv, b, a, gate, H, G, dk, dv, A_log, dt_bias, norm_w, eps)
    proj = torch.cat([b, torch.zeros(n, 3)], dim=1).to(dev)  # (the write strength's columns; the decay's are not read)
    consts = (A_log.to(dev), dt_bias.to(dev), norm_w.to(dev), eps)
    x, a_d, gate_d = qkv.to(dev), a.to(dev), gate.to(dev)
    state = torch.zeros((3, H * dv * dk + 4), device=dev)
    rows, slots = _rows(n, [], dev)
    kw = dict(gate_act="sigmoid")
    whole = ops.gated_delta(x, proj, 0, 0, 0, *consts, state, 4, rows, slots, H, G, dk, dv, gate=gate_d, channel_decay=a_d, **kw).cpu()
    assert (whole.double() - want).abs().max() < 3e-4 * want.abs().max(), (whole.double() - want).abs().max()
    state2 = torch.zeros_like(state)
    one_row = torch.tensor([1], dtype=torch.int32, device=dev)
    out, at = [], 0
    for m in [1, 1, 15, 16, 17, 2, 1, 33, 1, 64, 1, 1, 100, 1, 5, 1, 40]:
        out.append(ops.gated_delta(x[at : at + m].contiguous(), proj[at : at + m].contiguous(), 0, 0, 0, *consts, state2, 4,
                                   torch.tensor([0, m], dtype=torch.int32, device=dev), one_row, H, G, dk, dv,
                                   gate=gate_d[at : at + m].contiguous(), channel_decay=a_d[at : at + m].contiguous(), **kw).cpu())
        at += m
    assert at == n
    assert torch.equal(torch.cat(out), whole)
    assert torch.equal(state2[1], state[0])
    # one decay for the head would be another result altogether
    mean_a = a.reshape(n, H, dk).mean(-1, keepdim=True).expand(n, H, dk).reshape(n, H * dk)
    other = _plain_delta(qkv, b, mean_a, gate, H, G, dk, dv, A_log, dt_bias, norm_w, eps)
    assert (other - want).abs().max() > 0.1 * want.abs().max()


def test_router_kernel_and_experts_against_the_plain_functions():
    """Scores, the correction that changes the choice but not the weights, experts that hand their input through,
    one choice and all, and the experts' products over the rows that chose them (more rows than a block holds at
    once among them), with a shared expert's gate."""
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(4)
    for n_out, top in ((5, 2), (7, 7), (64, 1), (130, 9)):
        z = torch.randn((50, n_out + 1), generator=g) * 2
        corr = torch.randn(n_out, generator=g) * 0.5
        ids, wts = ops.router_topk(z.to(dev), n_out, corr.to(dev), top)
        s = torch.softmax(z[:, :n_out].double(), -1)
        want_ids = torch.topk(s + corr.double(), top).indices
        assert torch.equal(ids.cpu().long().sort(-1).values, want_ids.sort(-1).values)
        assert torch.allclose(wts.cpu().double(), s.gather(1, ids.cpu().long()), atol=1e-6)
        plain_choice = torch.topk(s, top).indices.sort(-1).values
        assert n_out == top or not torch.equal(plain_choice, want_ids.sort(-1).values)  # the correction matters
    # (many pairs: the matrix cores; few: a wave an output with its weights in registers)
    for n in (61, 2):
        D, F, E, I, top = 48, 40, 4, 2, 3
        x = torch.randn((n, D), generator=g)
        w_gu = torch.randn((E, 2 * F, D), generator=g) * 0.2
        w_d = torch.randn((E, D, F), generator=g) * 0.2
        ids = torch.stack([torch.randperm(E + I, generator=g)[:top] for _ in range(n)]).to(torch.int32)
        wts = torch.rand((n, top), generator=g)
        shared, sg = torch.randn((n, D), generator=g), torch.randn((n, 3), generator=g)
        for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 3e-2)):
            xd = x.to(dtype).to(dev)
            rows, pos, offsets = ops.expert_gather(xd, ids.to(dev), E + I)
            y = ops.expert_down_rows(ops.expert_glu_rows(rows, w_gu.to(dtype).to(dev), offsets), w_d.to(dtype).to(dev), offsets)
            got = ops.expert_combine(y, pos, ids.to(dev), wts.to(dev), E, xd, shared.to(dtype).to(dev), sg.to(dev)[:, 1])
            xr, gu, dn, sh = x.to(dtype).double(), w_gu.to(dtype).double(), w_d.to(dtype).double(), shared.to(dtype).double()
            want = plain.sigmoid(sg[:, 1:2].double()) * sh
            for t in range(n):
                for j in range(top):
                    e = int(ids[t, j])
                    y = xr[t] if e >= E else dn[e] @ (plain.silu(gu[e, :F] @ xr[t]) * (gu[e, F:] @ xr[t]))
                    want[t] += float(wts[t, j]) * y
            assert (got.double().cpu() - want).abs().max() < tol * want.abs().max()
            # the gathered rows themselves, and the same result through one matrix product per expert
            bounds = offsets.tolist()
            assert bounds[0] == 0 and bounds[-1] == n * top
            assert [bounds[e + 1] - bounds[e] for e in range(E + I)] == torch.bincount(ids.flatten().long(), minlength=E + I).tolist()
            assert sorted(pos.flatten().tolist()) == list(range(n * top))
            for t in range(n):
                for j in range(top):
                    at = int(pos[t, j])
                    assert bounds[int(ids[t, j])] <= at < bounds[int(ids[t, j]) + 1] and torch.equal(rows[at], xd[t])
            parts = [ops.linear(ops.linear_glu(rows[bounds[e] : bounds[e + 1]], w_gu.to(dtype).to(dev)[e]), w_d.to(dtype).to(dev)[e])
                     for e in range(E) if bounds[e + 1] > bounds[e]]
            again = ops.expert_combine(torch.cat(parts), pos, ids.to(dev), wts.to(dev), E, xd, shared.to(dtype).to(dev), sg.to(dev)[:, 1])
            assert (again.double().cpu() - want).abs().max() < 2 * tol * want.abs().max()
            if dtype == torch.bfloat16 and n * top <= 8:
                # and every pair by the weight-streaming products that read on the device which expert is meant
                y = ops.expert_pair_products(xd, w_gu.to(dtype).to(dev), w_d.to(dtype).to(dev), ids.to(dev))
                own = torch.arange(n * top, dtype=torch.int32, device=dev).view(n, top)
                third = ops.expert_combine(y, own, ids.to(dev), wts.to(dev), E, xd, shared.to(dtype).to(dev), sg.to(dev)[:, 1])
                assert (third.double().cpu() - want).abs().max() < 2 * tol * want.abs().max()


def test_norm_behind_a_branch_joined_with_the_next_norm():
    from torchllms_amd.kernels import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(2)
    for width in (64, 200, 1024, 5000):
        stream = torch.randn((9, width), generator=g) * 3
        branch = torch.randn((9, width), generator=g) * 0.1
        w1, w2 = torch.randn(width, generator=g), torch.randn(width, generator=g)
        new = stream.double() + plain.rms_unit(branch.double(), 1e-5) * w1.double()
        rows = plain.rms_unit(new, 1e-6) * w2.double()
        for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
            s = stream.clone().to(dev)
            y = ops.post_norm_add_norm(s, branch.to(dtype).to(dev), w1.to(dev), 1e-5, w2.to(dev), 1e-6)
            ref_new = stream.double() + plain.rms_unit(branch.to(dtype).double(), 1e-5) * w1.double()
            assert (s.cpu().double() - ref_new).abs().max() < 1e-5
            assert (y.cpu().double() - plain.rms_unit(ref_new, 1e-6) * w2.double()).abs().max() < tol * rows.abs().max()
            s2 = stream.clone().to(dev)
            assert ops.post_norm_add_norm(s2, branch.to(dtype).to(dev), w1.to(dev), 1e-5) is None
            assert torch.equal(s2, s)


# ----------------------------------------------------------------------------- far back, first tokens, slots used again
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_with_sharp_attention_and_long_memory(tmp_path, dtype):
    """Scores with a spread of four make every query look at a few keys anywhere in 700 tokens, forget gates near
    one keep what the first tokens wrote: a lost page, a key one off or a state that was not carried shows in the
    logits of late positions, whole, in portions that end at and beside page borders, and decoded one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = models.model(97, 64, 2.0, 1e-5, [
        models.layer("parallel", models.pair(models.left(4, 2, 32, 16, 0.3), models.right(2, 1, 32, 32, 4, 8, 8), 1.0, 0.6), models.dense(64)),
        models.layer("mlstm", models.mlstm(2, 32, 32, 15.0), models.moe(32, 4, 2, identity=1, shared=16)),
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
    assert at == 700
    cut = torch.cat(rows)
    for name, got in (("whole", whole), ("cut", cut)):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(700)]
        if dtype == "float32":
            assert max(dists) < tol, f"{name}: distance {max(dists)}"
        else:
            assert_within_rounding(dists, tol, name)
    if dtype == "float32":
        assert torch.equal(whole, cut)
    # dropping what lies far back would be seen: the truth of the last 100 tokens alone is another
    short = plain.forward(cfg, {k: v.double() for k, v in weights.items()}, tokens[600:])
    assert max(distance(short[i], truth["r"][600 + i], scale) for i in range(50, 100)) > 10 * tol


def test_a_slot_that_is_used_again_starts_from_zero(tmp_path):
    """One state slot and few pages: each request takes over what the one before left (the matrix memory with its
    maxima, the delta rule's state, the convolutions' histories, pages of keys), and must not see any of it."""
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
    """Three requests decode 150 tokens together: the steps are replayed from HIP graphs after the first few, the
    states move on with every replay, and the logits stay the plain model's."""
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
    w64 = {k: v.double() for k, v in weights.items()}
    prompts = [random_tokens(n, cfg["vocab"], 40 + n) for n in (5, 37, 1, 64, 22)]
    new = 20

    def plain_greedy(prompt):
        toks = list(prompt)
        for _ in range(new):
            toks.append(int(plain.forward(cfg, w64, toks)[-1].argmax()))
        return toks[len(prompt):]

    llm = LLM(str(folder), precision="float32", max_len=128, max_bsz=3, page_size=8, max_num_batched_tokens=24)
    results = llm.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=new)
    for p, r in zip(prompts, results):
        assert r.token_ids == plain_greedy(p)
    llm.engine.cache.check_invariants()
    assert llm.engine.cache.live == []
    llm16 = LLM(str(folder), precision="bfloat16", max_len=128, max_bsz=3, page_size=8)
    for p, r in zip(prompts, llm16.generate(prompt_token_ids=prompts, temperature=0.0, max_new_tokens=4)):
        logits = plain.forward(cfg, w64, p)[-1]
        assert logits[r.token_ids[0]] >= logits.max() - 0.05 * float(logits.std())


def test_a_preempted_request_starts_again_from_clean_state(tmp_path):
    """Too few pages for four requests: the scheduler takes the youngest off, gives its pages and its slot away and
    later computes it again from its prompt and what it had generated; the sampled tokens are those of the run with
    room for everybody."""
    from torchllms_amd.inference import LLM

    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=9)
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

    from torchllms_amd.config.kepevik import KepevikConfig
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
    written = write_model_folder(tmp_path / "written", KepevikConfig.from_dict(models.CONFIG_B), seed=7, dtype=torch.float32)
    cfg, weights = models.read_folder(written)
    w64 = {k: v.double() for k, v in weights.items()}
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(plain.forward(cfg, w64, toks)[-1].argmax()))
    assert got == toks[len(prompt):]


def test_trace_replay_program(tmp_path):
    """``bin/trace_run`` as a process: steps in, logits files out, the plain model's values."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parent.parent
    folder = models.make_folder(tmp_path / "m", models.CONFIG_C, seed=6)
    cfg, weights = models.read_folder(folder)
    requests = {"x": random_tokens(50, cfg["vocab"], 1), "y": random_tokens(90, cfg["vocab"], 2), "z": random_tokens(20, cfg["vocab"], 3)}
    truth, scale = truth_of(cfg, weights, requests)
    steps = schedules.mixed(requests, max_live=2)
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(root / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(out),
         "--max-tokens", str(schedules.max_live_tokens(steps))],
        input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(len(steps))]
    for step, rows in zip(steps, schedules.positions_of(steps)):
        got = torch.from_numpy(np.fromfile(out / f"{step['step']}.f32", dtype="<f4").reshape(len(rows), -1))
        for row, (rid, pos) in zip(got, rows):
            assert distance(row, truth[rid][pos], scale) < FP32_TOL


# ----------------------------------------------------------------------------- sizes that no vector load divides
ODD = {
    "width_100": models.model(301, 100, 1.5, 1e-6, [
        models.layer("parallel", models.pair(models.left(3, 1, 20, 6, 0.2), models.right(3, 3, 12, 20, 3, 3, 5), 0.6, 0.5),
                     models.moe(36, 5, 2, identity=1, shared=20)),
        models.layer("mlstm", models.mlstm(5, 12, 20, 15.0), models.dense(52)),
        models.layer("mlstm", models.mlstm(2, 30, 50, 15.0), models.moe(28, 3, 3, identity=4)),
    ]),
    "width_36": models.model(97, 36, 3.0, 1e-6, [
        models.layer("mlstm", models.mlstm(1, 10, 6, 4.0), models.moe(12, 9, 4, identity=4, shared=4)),
        models.layer("parallel", models.pair(models.left(9, 3, 8, 8, 0.35, base=1e6), models.right(4, 1, 10, 14, 4, 2, 2), 0.6, 0.5), None),
    ]),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD))
def test_widths_that_are_no_multiple_of_eight(tmp_path, name, dtype):
    """Rows of 100 and 36 channels, experts of 36, 28 and 12, heads of 20, 12, 10 and 8, more experts that hand their
    input through than experts: the kernels' forms for rows that no 16-byte load divides, a prompt whole and then a
    prompt with its last 50 tokens one by one."""
    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = ODD[name]
    folder = folder_for(dtype, tmp_path / name, cfg_dict, seed=3)
    tokens = random_tokens(150, cfg_dict["vocab"], 4)
    truth, scale = truth_of(*models.read_folder(folder), {"r": tokens})
    engine = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=40, max_seqs=2)
    engine.admit("a")
    whole = engine.step([StepEntry("a", tokens, list(range(150)))]).cpu()
    engine.admit("b")
    rows = [engine.step([StepEntry("b", tokens[:100], list(range(100)))]).cpu()]
    rows += [engine.step([StepEntry("b", [t], [0])]).cpu() for t in tokens[100:]]
    cut = torch.cat(rows)
    for got in (whole, cut):
        dists = [distance(got[i], truth["r"][i], scale) for i in range(150)]
        if dtype == "float32":
            assert max(dists) < FP32_TOL
        else:
            assert_within_rounding(dists, 1.5 * BF16_TOL, name)
    if dtype == "float32":
        assert torch.equal(whole, cut)


# ----------------------------------------------------------------------------- random configurations
def random_config(seed: int) -> dict:
    """A Kepevik configuration drawn from a seed: every size, constant and the order of layers."""
    import random

    rng = random.Random(seed)
    width = rng.choice([40, 64, 72, 96, 128, 160])
    layers = []
    for _ in range(rng.randint(2, 5)):
        mlp = rng.choice([None, models.dense(rng.choice([48, 100, 136])),
                          models.moe(rng.choice([16, 24, 40, 72]), rng.choice([1, 2, 5, 9]), 1, identity=rng.choice([None, 0, 1, 3]),
                                     shared=rng.choice([None, 16, 56]))])
        if mlp is not None and mlp["kind"] == "moe":
            r = mlp["router"]
            r["top"] = rng.randint(1, r["experts"] + (r.get("identity") or 0))
        if rng.random() < 0.5:
            mixer = models.mlstm(rng.choice([1, 2, 3, 4]), rng.choice([8, 20, 32, 64, 128, 192]), rng.choice([1, 8, 24, 31, 64, 100]),
                                 rng.choice([1.0, 5.0, 15.0, 40.0]))
            layers.append(models.layer("mlstm", mixer, mlp))
            continue
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([16, 24, 32, 64, 128])
        lf = models.left(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([0, dim // 2, dim]) // 2 * 2, rng.choice([0.1, 0.3, 1.0]) * 32 / dim,
                         base=rng.choice([100.0, 10000.0, 1000000.0]))
        kv = rng.choice([1, 2, 3])
        rt = models.right(kv * rng.choice([1, 2]), kv, rng.choice([8, 20, 32, 64, 128, 192]), rng.choice([8, 24, 32, 64, 100]),
                          rng.choice([1, 2, 3, 4, 5]), rng.choice([1, 4, 24]), rng.choice([2, 8, 24]))
        layers.append(models.layer("parallel", models.pair(lf, rt, rng.choice([0.3, 0.6, 1.0]), rng.choice([0.5, 1.0, 1.4])), mlp))
    return models.model(rng.choice([50, 97, 256, 301]), width, rng.choice([1.0, 0.5, 12.0]), rng.choice([1e-5, 1e-6, 1e-3]), layers)


@pytest.mark.parametrize("seed", range(8))
def test_random_configurations(tmp_path, seed):
    """Sizes nobody chose: a prompt whole, and the same tokens in portions, single tokens and beside a second
    request, in both dtypes, against the plain model."""
    import random

    from torchllms_amd.engine import Engine, StepEntry

    cfg_dict = random_config(2000 + seed)
    rng = random.Random(seed)
    requests = {"a": random_tokens(rng.randint(120, 330), cfg_dict["vocab"], seed), "b": random_tokens(rng.randint(20, 90), cfg_dict["vocab"], seed + 50)}
    page = rng.choice([4, 8, 16, 32])
    for dtype, tol in (("float32", FP32_TOL), ("bfloat16", 5 * BF16_TOL)):
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
