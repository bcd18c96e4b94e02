"""The Kepevik decoder without a GPU: its configuration, the model it describes, the tensor names, the sizes that
the tensors' shapes give, and the plain implementation's mechanisms against each other."""

import copy
import json

import pytest
import torch

from . import kepevik_models as models
from .helpers import random_tokens
from .plain import kepevik as plain


def test_configuration_round_trip_and_refusals():
    from torchllms_amd.config import ConfigError
    from torchllms_amd.config.kepevik import KepevikConfig

    for cfg_dict in models.CONFIGS.values():
        cfg = KepevikConfig.from_dict(cfg_dict)
        again = KepevikConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
        assert again == cfg
        assert len(cfg.layers) == len(cfg_dict["layers"])

    def broken(change):
        d = copy.deepcopy(models.CONFIG_A)
        change(d)
        with pytest.raises(ConfigError):
            KepevikConfig.from_dict(d)

    broken(lambda d: d["layers"][0].update(type="attention"))
    broken(lambda d: d["layers"][0]["mixer"]["left"].update(vdim=48))  # the values are the keys
    broken(lambda d: d["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda d: d["layers"][0]["mixer"]["left"]["rot"].update(dims=7))
    broken(lambda d: d["layers"][0]["mixer"].pop("right_scale"))
    broken(lambda d: d["layers"][1]["mixer"].update(gate_cap=0.0))
    broken(lambda d: d["layers"][0]["mlp"]["router"].update(top=9))
    broken(lambda d: d["layers"][1]["mlp"].update(kind="glu"))
    broken(lambda d: d.pop("norm"))


def test_model_spec_names_the_parts_and_the_tensors_round_trip(tmp_path):
    from torchllms_amd.config import load_config
    from torchllms_amd.parts.model import Model

    folder = models.make_folder(tmp_path / "m", models.CONFIG_A, seed=2)
    arch, cfg = load_config(folder)
    assert arch.name == "Kepevik"
    spec = arch.model_spec(cfg)
    assert [l.block for l in spec.layers] == ["sandwich_pair", "sandwich", "sandwich", "sandwich_pair_mixer"]
    assert spec.head.params["tied"] and spec.embedding.params["scale"] == 2.0
    model = Model(spec)
    needs = dict(model.cache_needs())
    assert type(needs[(0, "left")]).__name__ == "KVNeed" and type(needs[(0, "right")]).__name__ == "StateNeed"
    assert type(needs[(1, "mix")]).__name__ == "StateNeed"
    _, tensors = models.read_folder(folder)
    assert "l0.mix.left.v" not in tensors and "head" not in tensors
    assert tensors["l0.mix.right.a1"].shape == (6, 64) and tensors["l0.mix.right.g2"].shape == (4 * 32, 10)
    assert tensors["l2.mlp.router"].shape == (4, 64) and "l2.mlp.shared.sg" not in tensors
    assert tensors["l0.mlp.router"].shape == (7, 64) and tensors["l0.mlp.shared.sg"].shape == (1, 64)
    assert "l3.norm2" not in tensors and "l3.ls2" not in tensors and tensors["l3.ls1"].shape == (64,)


def test_sizes_that_only_the_tensors_give(tmp_path):
    """config.json need not say how many numbers lie between the two matrices of the decay and of the gate: the
    shapes of ``a1`` and ``g1`` do, and a folder whose configuration is silent loads with them."""
    from torchllms_amd.config import load_config

    folder = models.make_folder(tmp_path / "m", models.CONFIG_C, seed=3)
    cfg_dict = json.loads((folder / "config.json").read_text())
    for layer in cfg_dict["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop("decay_rank")
            layer["mixer"]["right"].pop("gate_rank")
    (folder / "config.json").write_text(json.dumps(cfg_dict))
    _, cfg = load_config(folder)
    assert cfg.layers[0].mixer["right"]["decay_rank"] == 16 and cfg.layers[0].mixer["right"]["gate_rank"] == 8
    assert cfg.layers[1].mixer["right"]["decay_rank"] == 8 and cfg.layers[1].mixer["right"]["gate_rank"] == 24


# ----------------------------------------------------------------------------- the plain model against itself
def _weights(cfg_dict, tmp_path, seed=1, **kw):
    folder = models.make_folder(tmp_path / f"w{seed}", cfg_dict, seed=seed, dtype=torch.float32, **kw)
    cfg, tensors = models.read_folder(folder)
    return cfg, {k: v.double() for k, v in tensors.items()}


def test_plain_model_is_causal(tmp_path):
    cfg, w = _weights(models.CONFIG_A, tmp_path)
    toks = random_tokens(40, cfg["vocab"], 3)
    full = plain.forward(cfg, w, toks)
    part = plain.forward(cfg, w, toks[:25])
    assert torch.allclose(full[:25], part, atol=1e-9)
    other = plain.forward(cfg, w, toks[:30] + [(t + 1) % cfg["vocab"] for t in toks[30:]])
    assert torch.allclose(full[:30], other[:30], atol=1e-9) and not torch.allclose(full[30:], other[30:], atol=1e-3)


def test_plain_matrix_memory_against_its_unrolled_sum():
    """Without the running maximum the cell is a weighted sum over the past: C_t = sum_s exp(i_s + F_t - F_s) k_s v_s^T
    with F the running sum of the log forget gates; the stabilised recurrence must give the same read-out, with the
    denominator's floor exp(-m) turned into a floor of 1 on the unstabilised scale."""
    torch.manual_seed(0)
    S, D, H, dk, dv, cap, eps = 30, 12, 2, 5, 7, 4.0, 1e-5
    m = {"heads": H, "dim": dk, "vdim": dv, "gate_cap": cap}
    w = {"x." + n: torch.randn(shape, dtype=torch.float64) for n, shape in
         dict(q=(H * dk, D), k=(H * dk, D), v=(H * dv, D), g=(H * dv, D), o=(D, H * dv), i=(H, D), f=(H, D)).items()}
    w["x.i.b"] = torch.randn(H, dtype=torch.float64)
    w["x.f.b"] = torch.randn(H, dtype=torch.float64) + 1.0
    w["x.norm"] = torch.rand(H * dv, dtype=torch.float64) + 0.5
    h = torch.randn(S, D, dtype=torch.float64)
    got = plain.matrix_memory(h, w, "x.", m, eps)
    q = (h @ w["x.q"].T).reshape(S, H, dk) * dk ** -0.5
    k = (h @ w["x.k"].T).reshape(S, H, dk)
    v = (h @ w["x.v"].T).reshape(S, H, dv)
    gi = cap * torch.tanh((h @ w["x.i"].T + w["x.i.b"]) / cap)
    gf = plain.log_sigmoid(cap * torch.tanh((h @ w["x.f"].T + w["x.f.b"]) / cap))
    F = gf.cumsum(0)
    out = torch.zeros(S, H, dv, dtype=torch.float64)
    for a in range(H):
        for t in range(S):
            wts = torch.exp(gi[: t + 1, a] + F[t, a] - F[: t + 1, a])
            num = ((wts * (k[: t + 1, a] @ q[t, a]))[:, None] * v[: t + 1, a]).sum(0)
            nq = (wts * (k[: t + 1, a] @ q[t, a])).sum()
            # m_t = max over s of (i_s + F_t - F_s) and of F_t (the start, m_0 = 0)
            mt = torch.maximum((gi[: t + 1, a] + F[t, a] - F[: t + 1, a]).max(), F[t, a])
            out[t, a] = num * torch.exp(-mt) / (torch.maximum(nq.abs() * torch.exp(-mt), torch.exp(-mt)) + 1e-6)
    want = plain.rms_unit(out, eps).reshape(S, H * dv) * w["x.norm"] * plain.sigmoid(h @ w["x.g"].T)
    assert torch.allclose(got, want @ w["x.o"].T, atol=1e-9)


def test_plain_router_counts_identity_experts_and_keeps_scores_unnormalised(tmp_path):
    cfg, w = _weights(models.single_layer(models.layer("mlstm", models.mlstm(1, 4, 4, 5.0), models.moe(16, 3, 2, identity=2))), tmp_path)
    h = torch.randn(9, cfg["width"], dtype=torch.float64)
    mlp = cfg["layers"][0]["mlp"]
    # with a correction that forces the two identity experts, the result is the input times their two scores
    w2 = dict(w)
    w2["l0.mlp.correction"] = torch.tensor([-9.0, -9.0, -9.0, 9.0, 9.0], dtype=torch.float64)
    s = torch.softmax(h @ w["l0.mlp.router"].T, -1)
    assert torch.allclose(plain.routed(h, w2, "l0.mlp.", mlp), h * (s[:, 3] + s[:, 4])[:, None], atol=1e-12)
    # and with one that forces experts 0 and 2, their outputs times their scores
    w2["l0.mlp.correction"] = torch.tensor([9.0, -9.0, 9.0, -9.0, -9.0], dtype=torch.float64)
    want = s[:, 0:1] * plain.gated_expert(h, w, "l0.mlp.e0.") + s[:, 2:3] * plain.gated_expert(h, w, "l0.mlp.e2.")
    assert torch.allclose(plain.routed(h, w2, "l0.mlp.", mlp), want, atol=1e-12)
