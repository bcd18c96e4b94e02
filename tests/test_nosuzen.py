"""Nosuzen without a GPU: the configuration and what it refuses, tensor names there and back, the cache's handling of
first positions that a window keeps and of a mixer that keeps pages and state, and the plain implementation pinned
by what fixes it beside its own text."""

import json
import math

import pytest
import torch

from torchllms_amd.cache.manager import CacheManager, group_layers
from torchllms_amd.config import ConfigError, load_config
from torchllms_amd.config.nosuzen import NosuzenConfig, nosuzen_model_spec
from torchllms_amd.parts.base import KVNeed
from torchllms_amd.parts.model import Model
from torchllms_amd.parts.positions import rotary_inverse_frequencies, yarn_magnitude

from . import nosuzen_models as models
from .plain import nosuzen as plain


@pytest.mark.parametrize("name", sorted(models.CONFIGS))
def test_configuration_there_and_back(name):
    cfg = NosuzenConfig.from_dict(models.CONFIGS[name])
    again = NosuzenConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
    assert again == cfg
    spec = nosuzen_model_spec(cfg)
    assert len(spec.layers) == len(cfg.layers) and spec.vocab_size == cfg.vocab
    for run, layer in zip(spec.order, cfg.layers):
        assert run.cache_from == (layer.mixer.get("kv_from") if layer.type == "attention" else None)


def _with(cfg, path, value):
    d = json.loads(json.dumps(cfg))
    at = d
    for key in path[:-1]:
        at = at[key]
    if value is None:
        at.pop(path[-1], None)
    else:
        at[path[-1]] = value
    return d


@pytest.mark.parametrize("path,value", [
    (("streams",), 0), (("streams",), None), (("layers", 0, "type"), "mlstm"), (("layers", 0, "mixer", "heads"), 3),
    (("layers", 0, "mixer", "rot", "dims"), 18), (("layers", 0, "mixer", "rot", "dims"), 7), (("layers", 0, "mixer", "mask"), {}),
    (("layers", 0, "mixer", "mask", "keep_first"), -1), (("layers", 0, "mlp", "router", "groups", "count"), 4),
    (("layers", 0, "mlp", "router", "groups", "keep"), 4), (("layers", 0, "mlp", "router", "top"), 9),
    (("layers", 1, "mixer", "rot", "dims"), 4), (("layers", 1, "mixer", "rot", "scaling"), {"factor": 2.0}),
    (("layers", 2, "mixer", "right", "tau"), 0.0), (("layers", 2, "mixer", "left_scale"), None),
    (("layers", 3, "mixer", "kv_from"), 3), (("layers", 3, "mixer", "kv_from"), 1), (("layers", 3, "mixer", "vdim"), 16),
    (("layers", 0, "mlp", "kind"), "dense"), (("norm",), {"eps": 0}),
])
def test_configuration_refuses(path, value):
    with pytest.raises(ConfigError):
        NosuzenConfig.from_dict(_with(models.CONFIG_A, path, value))


def test_a_layer_may_not_read_a_layer_that_reads():
    d = _with(models.CONFIG_B, ("layers", 3), dict(models.CONFIG_B["layers"][2], mixer=dict(models.CONFIG_B["layers"][2]["mixer"], kv_from=2)))
    with pytest.raises(ConfigError):
        NosuzenConfig.from_dict(d)


def test_folder_there_and_back_and_the_size_the_tensors_give(tmp_path):
    """``write_model_folder`` names every tensor as a checkpoint does, the loader finds every one again, and the number
    of values between the two matrices of the linear attention's decay is read off the tensors when config.json is
    silent about it."""
    from safetensors.torch import load_file

    from torchllms_amd.weights import load_weights, write_model_folder

    cfg = NosuzenConfig.from_dict(models.CONFIG_A)
    folder = write_model_folder(tmp_path / "m", cfg, seed=1, dtype=torch.float32)
    names = set(load_file(str(folder / "model.safetensors")))
    assert {"embed", "head", "final.norm", "final.norm.b", "final.norm.alpha", "l0.hc1.in", "l0.hc2.mix", "l0.mix.q.conv", "l0.mix.lq1",
            "l1.mix.dkv.norm", "l1.hc1.out", "l2.mix.left.q.norm", "l2.mix.right.a2.b", "l2.mlp.e3.down", "l0.mlp.shared.up",
            "l3.mix.q", "l3.mix.q.conv"} <= names
    assert not {"l1.hc2.in", "l1.norm2", "l3.mix.k", "l3.mix.v.conv", "l2.mlp.shared.up", "l0.mlp.correction"} & names
    raw = json.loads((folder / "config.json").read_text())
    del raw["layers"][2]["mixer"]["right"]["decay_rank"]
    (folder / "config.json").write_text(json.dumps(raw))
    arch, loaded = load_config(folder)
    assert arch.name == "Nosuzen" and loaded.layers[2].mixer["right"]["decay_rank"] == 6
    model = Model(arch.model_spec(loaded))
    tensors = load_weights(folder, arch.weight_rules(loaded), model.param_specs(), torch.float32, device="cpu")
    assert set(tensors) == set(model.param_specs())
    model.bind(tensors)


def test_cache_entries_of_a_mixer_with_pages_and_state():
    """Differential attention keeps pages and the convolutions' histories; a layer that reads another's pages keeps a
    history of its own (of its queries alone); the pages of the owner serve the widest mask of all readers."""
    model = Model(nosuzen_model_spec(NosuzenConfig.from_dict(models.CONFIG_A)))
    keys = {key: need for key, need in model.cache_needs()}
    assert set(keys) == {(0, "mix", "kv"), (0, "mix", "conv"), (1, "mix"), (2, "left"), (2, "right"), (3, "mix", "conv")}
    kv = keys[(0, "mix", "kv")]
    assert (kv.num_kv_heads, kv.num_v_heads, kv.head_dim, kv.v_head_dim) == (4, 2, 16, 24)
    assert (kv.window, kv.keep_first) == (40, 5)  # layer 3 reads them through a window of 40, layer 0 keeps five positions
    assert keys[(0, "mix", "conv")].shape == (3 * (4 * 2 * 16 + 2 * 2 * 16 + 2 * 24),)
    assert keys[(3, "mix", "conv")].shape == (1 * 4 * 2 * 16,)
    assert model._run_caches[3] == [("mix", "conv", (3, "mix", "conv"), True), ("mix", "kv", (0, "mix", "kv"), False)]
    groups, states = group_layers(model.cache_needs())
    assert sorted((g.window, g.keep_first) for g in groups) == [(20, 3), (30, 0), (40, 5)]
    assert len(states) == 3
    # a reader without a window keeps every page of the owner
    from torchllms_amd.parts.attention import covering_window

    assert covering_window([(24, 5), (0, 0)]) == (0, 0) and covering_window([(24, 5), (40, 0), (8, 9)]) == (40, 9)


def test_pages_of_kept_first_positions_stay():
    need = KVNeed(num_kv_heads=2, head_dim=8, window=10, keep_first=5)
    groups, states = group_layers([(("r", "kv"), need)])
    cache = CacheManager(groups, states, page_size=4, num_pages=12, max_seqs=2)
    assert cache.kept_blocks(0) == 2
    cache.admit("a")
    for n in (3, 9, 1, 1, 20, 1, 1, 1):
        cache.extend("a", n)
        cache.advance("a", n)
        cache.check_invariants()
    table = cache.block_table("a")
    held = cache.num_tokens("a")
    first_needed = (held - 10 + 1) // 4
    assert all(p >= 0 for p in table[:2]) and all(p == -1 for p in table[2:first_needed]) and all(p >= 0 for p in table[first_needed:])
    cache.free("a")
    cache.check_invariants()
    assert cache.free_pages(0) == 12
    # without a window nothing is kept apart: every page stays anyway
    groups, _ = group_layers([(("r", "kv"), KVNeed(num_kv_heads=2, head_dim=8, window=0, keep_first=5))])
    assert groups[0].keep_first == 0


def test_the_scheduler_counts_the_kept_pages():
    from torchllms_amd.engine.scheduler import Scheduler

    groups, states = group_layers([(("r", "kv"), KVNeed(num_kv_heads=1, head_dim=8, window=16, keep_first=9))])
    cache = CacheManager(groups, states, page_size=4, num_pages=100, max_seqs=2)

    class Fake:
        pass

    fake = Fake()
    fake.cache = cache
    assert Scheduler._most_pages_held(fake, 0, 1000) == 4 + 1 + 3
    assert Scheduler._most_pages_held(fake, 0, 10) == 3


# ----------------------------------------------------------------------------- the plain implementation, pinned
def test_plain_mask_by_hand():
    m = plain.visible(9, 3, 2)
    assert m[8].tolist() == [True, True, False, False, False, False, True, True, True]
    assert m[3].tolist() == [True, True, True, True, False, False, False, False, False]
    assert plain.visible(5, 1)[4].tolist() == [False, False, False, False, True]


def test_plain_rotation_layouts_and_relative_positions():
    """Both layouts rotate each pair by the same angle, scores depend on the distance alone, the rest passes."""
    rot = {"dims": 8, "base": 100.0}
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn((1, 12), generator=g, dtype=torch.float64), torch.randn((1, 12), generator=g, dtype=torch.float64)
    for layout in ("half", "interleaved"):
        a = (plain.rotate(q, torch.tensor([7]), rot, layout) * plain.rotate(k, torch.tensor([3]), rot, layout)).sum()
        b = (plain.rotate(q, torch.tensor([104]), rot, layout) * plain.rotate(k, torch.tensor([100]), rot, layout)).sum()
        assert abs(a - b) < 1e-9
        assert torch.equal(plain.rotate(q, torch.tensor([5]), rot, layout)[:, 8:], q[:, 8:])
    half = plain.rotate(q, torch.tensor([1]), rot, "half")
    inter = plain.rotate(q[:, [0, 4, 1, 5, 2, 6, 3, 7, 8, 9, 10, 11]], torch.tensor([1]), rot, "interleaved")
    assert torch.allclose(half[:, [0, 4, 1, 5, 2, 6, 3, 7]], inter[:, :8])
    assert abs(half[0, 0] - (q[0, 0] * math.cos(1.0) - q[0, 4] * math.sin(1.0))) < 1e-12


def test_yarn_by_hand_and_in_the_engine():
    """dims 8, base 100, original 64, fast 4, slow 1: pair i turns 64 / (2 pi 100^(i/4)) times; the ramp runs from
    floor(0.81) = 0 to ceil(2.01) = 3."""
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 4.0, "slow": 1.0}}
    f, mag = plain.rotary_frequencies(rot)
    base = [100.0 ** (-i / 4) for i in range(4)]
    ramp = [0.0, 1 / 3, 2 / 3, 1.0]
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    assert f.tolist() == pytest.approx([b / 4.0 * r + b * (1 - r) for b, r in zip(base, ramp)])
    scaling = dict(rot["scaling"], rope_type="yarn")
    assert rotary_inverse_frequencies(8, 100.0, scaling).double().tolist() == pytest.approx(f.tolist(), rel=1e-6)
    assert yarn_magnitude(scaling) == pytest.approx(mag) and yarn_magnitude(None) == 1.0


def test_plain_convolution_and_linear_attention_step_by_step():
    u = torch.arange(10, dtype=torch.float64).reshape(5, 2) + 1
    taps = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 2.0]], dtype=torch.float64)
    y = plain.short_conv(u, taps)
    assert y[0].tolist() == [100.0, 4.0] and y[1].tolist() == [310.0, 8.0] and y[4].tolist() == [5 + 70 + 900, 20.0]
    # linear attention with one head and one channel: S_t = alpha S + k v, o = S q / 1
    w = {"p.q": torch.tensor([[1.0]]), "p.k": torch.tensor([[2.0]]), "p.v": torch.tensor([[3.0]]), "p.g": torch.tensor([[1.0]]),
         "p.a1": torch.tensor([[0.0]]), "p.a2": torch.tensor([[0.0]]), "p.a2.b": torch.tensor([0.0]), "p.norm": torch.tensor([1.0]),
         "p.o": torch.tensor([[1.0]])}
    w = {k: v.double() for k, v in w.items()}
    h = torch.tensor([[1.0], [1.0], [1.0]], dtype=torch.float64)
    out = plain.gated_linear_attention(h, w, "p.", {"heads": 1, "dim": 1, "vdim": 1, "tau": 1.0}, 0.0)
    # alpha = 1/2: S = 6, 9, 10.5; o = S; normed to 1, times silu(1)
    assert out[:, 0].tolist() == pytest.approx([float(plain.silu(torch.tensor(1.0)))] * 3)


def test_plain_router_by_hand():
    z = torch.log(torch.tensor([[0.30, 0.05, 0.25, 0.40]], dtype=torch.float64))
    ids, w = plain.routed_choice(z, {"experts": 4, "top": 2, "scale": 3.0})
    assert ids.tolist() == [[3, 0]] and w[0].tolist() == pytest.approx([3 * 0.4 / 0.7, 3 * 0.3 / 0.7])
    ids, w = plain.routed_choice(z, {"experts": 4, "top": 2, "scale": 1.0, "groups": {"count": 2, "keep": 1}})
    assert ids.tolist() == [[3, 2]] and w[0].tolist() == pytest.approx([0.4 / 0.65, 0.25 / 0.65])


def test_plain_streams_by_hand():
    x = torch.tensor([[[1.0]], [[2.0]]], dtype=torch.float64)  # two streams, one token, one channel
    w = {"h.in": torch.tensor([1.0, -1.0]), "h.out": torch.tensor([10.0, 100.0]), "h.mix": torch.tensor([[1.0, 2.0], [3.0, 4.0]]),
         "n": torch.tensor([2.0]), "n.b": torch.tensor([0.5]), "n.alpha": torch.tensor(1.0)}
    w = {k: v.double() for k, v in w.items()}
    seen = []
    out = plain.hyper_sublayer(x, w, "h", "n", lambda h: (seen.append(h.clone()), h * 0 + 1.0)[1])
    assert seen[0].item() == pytest.approx(math.tanh(-1.0) * 2.0 + 0.5)
    assert out[:, 0, 0].tolist() == [1 * 1 + 3 * 2 + 10, 2 * 1 + 4 * 2 + 100]
