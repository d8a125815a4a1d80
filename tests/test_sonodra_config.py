"""Sonodra's configuration, plan, cache needs and model folder: what runs without a GPU."""
import copy
import json
import os

import pytest
import torch

import plain_sonodra as ps
from sonodra_cases import CONFIGS, settled_tokens, write_folder


def test_configuration_round_trip_and_plan():
    from bitnet_c_amd.config import SonodraConfig, architecture_for
    from bitnet_c_amd.config.sonodra import build_sonodra_plan
    for name, raw in CONFIGS.items():
        assert architecture_for(raw).name == "Sonodra"
        c = SonodraConfig.from_dict(raw)
        assert SonodraConfig.from_dict(c.to_dict()) == c
        assert c.to_dict()["layers"] == raw["layers"]
        plan = build_sonodra_plan(c)
        assert len(plan.layers) == len(plan.schedule) == len(raw["layers"])
        D = raw["width"]
        t = plan.expected_tensors()
        assert t["embed"].shape == (raw["vocab"], D) == t["head"].shape and t["final.norm"].shape == (D,)
        for i, (e, L) in enumerate(zip(plan.schedule, raw["layers"])):
            p, m = f"l{i}.", L["mixer"]
            assert e.layer == i and e.kv_from == m.get("kv_from")
            assert t[p + "norm1"].shape == t[p + "norm1b"].shape == (D,)
            if L["type"] == "attention":
                assert t[p + "mix.q"].shape == (m["heads"] * m["dim"], D) and t[p + "mix.k"].shape == (m["kv_heads"] * m["dim"], D)
                assert t[p + "mix.v"].shape == (m["kv_heads"] * m["vdim"], D) and t[p + "mix.o"].shape == (D, m["heads"] * m["vdim"])
                assert t[p + "mix.q.norm"].shape == (m["heads"] * m["dim"],) and t[p + "mix.k.norm"].shape == (m["kv_heads"] * m["dim"],)
            else:
                assert t[p + "mix.q"].shape == (m["heads"] * m["dim"], D) and t[p + "mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
                assert t[p + "mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"]) == t[p + "mix.g"].shape[:1] + (m["kv_rank"],)
                assert t[p + "mix.g"].shape == (m["heads"] * m["vdim"], D) and t[p + "mix.o"].shape == (D, m["heads"] * m["vdim"])
                assert (p + "mix.dkv" in t) == (p + "mix.dkv.norm" in t) == ("kv_from" not in m)
                if "kv_from" not in m:
                    assert t[p + "mix.dkv"].shape == (m["kv_rank"], D) and t[p + "mix.dkv.norm"].shape == (m["kv_rank"],)
            mlp = L["mlp"]
            assert (p + "norm2" in t) == (p + "norm2b" in t) == (mlp is not None)
            if mlp is None:
                assert not [n for n in t if n.startswith(p + "mlp.")]
            elif mlp["kind"] == "dense":
                assert t[p + "mlp.gate"].shape == t[p + "mlp.up"].shape == (mlp["ff"], D) and t[p + "mlp.down"].shape == (D, mlp["ff"])
            else:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                assert t[p + "mlp.router"].shape == (E, D)
                assert sorted(n for n in t if n.startswith(p + "mlp.e")) == sorted(
                    f"{p}mlp.e{e}.{w}" for e in range(E) for w in ("up", "down"))
                assert t[f"{p}mlp.e{E - 1}.up"].shape == (F, D) and t[f"{p}mlp.e0.down"].shape == (D, F)


def _bad(raw, change, match):
    from bitnet_c_amd.config import ConfigError, SonodraConfig
    raw = copy.deepcopy(raw)
    change(raw)
    with pytest.raises(ConfigError, match=match):
        SonodraConfig.from_dict(raw)


def test_configurations_that_cannot_be_are_refused():
    A, B = CONFIGS["A"], CONFIGS["B"]
    _bad(A, lambda r: r["layers"][0].update(type="conv"), "type")
    _bad(A, lambda r: r["layers"][0]["mixer"].update(kv_heads=3), "kv_heads")
    _bad(A, lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims")
    _bad(A, lambda r: r["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims")
    _bad(A, lambda r: r["layers"][0]["mixer"].pop("scale"), "scale")
    _bad(A, lambda r: r["layers"][0]["mlp"].update(kind="glu"), "kind")
    _bad(A, lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "top")
    _bad(A, lambda r: r["layers"][2]["mixer"].update(kv_from=2), "kv_from")
    _bad(A, lambda r: r["layers"][2]["mixer"].update(kv_from=0), "keeps none")          # an attention layer has no latent
    _bad(A, lambda r: r["layers"][2]["mixer"].update(kv_rank=16), "kv_rank")
    _bad(A, lambda r: r["layers"][1]["mixer"].update(kv_from=2), "after it|keeps none")
    _bad(B, lambda r: r["layers"][3]["mixer"].update(kv_from=9), "kv_from")
    _bad(A, lambda r: r.pop("norm"), "norm")
    _bad(A, lambda r: r.update(layers=[]), "layers")


def test_cache_needs_windows_latents_and_shared_entries():
    """Attention layers keep keys and values of their own sizes and windows (layers of equal need share a group of pages),
    a latent layer keeps one head as wide as its latent, once as keys and once as values, and a layer that reads another's
    latent vectors has the other's pages and writes nothing."""
    from bitnet_c_amd.cache import PAGE, PagedCache
    from bitnet_c_amd.config import SonodraConfig
    from bitnet_c_amd.config.sonodra import build_sonodra_plan
    from bitnet_c_amd.parts import BLOCKS
    raw = CONFIGS["C"]
    plan = build_sonodra_plan(SonodraConfig.from_dict(raw))
    needs = [BLOCKS.build(plan.layers[e.layer].block).cache_need() for e in plan.schedule]
    for need, L in zip(needs, raw["layers"]):
        m = L["mixer"]
        assert need.state is None
        if L["type"] == "attention":
            assert (need.kv.n_kv_heads, need.kv.head_dim, need.kv.v_dim, need.kv.window) == (m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"])
        else:
            assert (need.kv.n_kv_heads, need.kv.head_dim, need.kv.v_dim, need.kv.window) == (1, m["kv_rank"], m["kv_rank"], 0)
    cache = PagedCache(needs, [e.kv_from for e in plan.schedule], 16 * PAGE)
    assert len(cache.groups) == 3 and cache.group_of(3) == cache.group_of(1) == cache.group_of(4)
    tables = {g: None for g in range(3)}
    assert cache.view(1, tables, 0).writes and not cache.view(3, tables, 0).writes and not cache.view(4, tables, 0).writes
    # a windowed group gives pages back while a sequence grows, the latent group keeps them all
    s = cache.alloc_slot()
    cache.reserve([s], [5 * PAGE])
    cache.commit([s], [5 * PAGE])
    held = {cache.groups[g].need.window: sum(p >= 0 for p in cache.pages_of(g, s)) for g in range(3)}
    assert held == {0: 5, 64: 1, 100: 2}
    cache.free_slot(s)
    cache.check()


def test_random_weights_folder_and_plain_reading(tmp_path):
    """The library writes a folder from a configuration alone; the plain implementation reads it and runs."""
    from bitnet_c_amd.config import SonodraConfig, load_config
    from bitnet_c_amd.weights import write_model_folder
    folder = write_model_folder(str(tmp_path / "made"), SonodraConfig.from_dict(CONFIGS["B"]), 5, torch.bfloat16)
    arch, cfg = load_config(folder)
    assert arch.name == "Sonodra" and cfg == SonodraConfig.from_dict(CONFIGS["B"])
    logits = ps.forward(ps.read_config(folder), ps.read_weights(folder), [1, 2, 3, 4])
    assert logits.shape == (4, 77) and bool(torch.isfinite(logits).all())


def test_a_folder_with_a_tensor_missing_or_left_over_is_refused(tmp_path):
    from safetensors.torch import load_file
    from bitnet_c_amd.config import SonodraConfig
    from bitnet_c_amd.config.sonodra import build_sonodra_plan
    from bitnet_c_amd.weights import WeightError, open_tensors, write_file
    folder = write_folder(tmp_path / "m", CONFIGS["A"], 1)
    plan = build_sonodra_plan(SonodraConfig.from_dict(CONFIGS["A"]))
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    tensors["l2.mix.dkv"] = tensors.pop("l1.mix.dkv")               # the reading layer has no down-projection
    tensors["l1.mlp.e5.up"] = tensors["l1.mlp.e5.up"][:-1].contiguous()
    write_file(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.raises(WeightError) as err:
        open_tensors(folder, plan.expected_tensors())
    assert err.value.missing == ["l1.mix.dkv"] and err.value.unexpected == ["l2.mix.dkv"]
    assert [n for n, _, _ in err.value.wrong_shape] == ["l1.mlp.e5.up"]


def test_the_plain_mechanisms_on_cases_worked_by_hand():
    """The oracle itself, where a result can be written down: a window of one token returns the token's own value, a
    rotation at position 0 changes nothing and keeps lengths anywhere, one expert with score s computes on s h."""
    g = torch.Generator().manual_seed(0)
    T, D = 5, 8
    h = torch.randn(T, D, generator=g, dtype=torch.float64)
    W = {"q": torch.randn(4, D, generator=g, dtype=torch.float64), "k": torch.randn(4, D, generator=g, dtype=torch.float64),
         "v": torch.randn(6, D, generator=g, dtype=torch.float64), "o": torch.eye(6, dtype=torch.float64),
         "q.norm": torch.ones(4, dtype=torch.float64), "k.norm": torch.ones(4, dtype=torch.float64)}
    m = dict(heads=1, kv_heads=1, dim=4, vdim=6, scale=0.5, mask=dict(size=1), rot=dict(base=10.0, dims=4))
    assert torch.allclose(ps.window_attention(h, W, "", m, 1e-6), h @ W["v"].T)
    x = torch.randn(3, 2, 6, generator=g, dtype=torch.float64)
    r = ps.rotate_pairs(x, [0, 3, 11], 4, 100.0)
    assert torch.equal(r[0], x[0]) and torch.equal(r[..., 4:], x[..., 4:])
    assert torch.allclose(r[..., :4].pow(2).sum(-1), x[..., :4].pow(2).sum(-1))
    assert torch.allclose(r[1, 0, 0], x[1, 0, 0] * torch.cos(torch.tensor(3.0, dtype=torch.float64)) - x[1, 0, 1] * torch.sin(torch.tensor(3.0, dtype=torch.float64)))
    Wm = {"router": torch.full((1, D), 0.1, dtype=torch.float64), "e0.up": torch.randn(3, D, generator=g, dtype=torch.float64),
          "e0.down": torch.randn(D, 3, generator=g, dtype=torch.float64)}
    y = ps.moe_ffn(h, Wm, "", dict(router=dict(experts=1, top=1)))
    s = ps.sigmoid(h @ Wm["router"].T)
    assert torch.allclose(y, (torch.clamp((s * h) @ Wm["e0.up"].T, min=0) ** 2) @ Wm["e0.down"].T)


def test_settled_sequences_have_no_close_expert_choice(tmp_path):
    folder = write_folder(tmp_path / "m", CONFIGS["A"], 2)
    toks = settled_tokens(folder, 60, 4)
    assert settled_tokens(folder, 40, 4) == toks[:40]
    margins = []
    ps.forward(ps.read_config(folder), ps.read_weights(folder), toks, margins=margins)
    assert len(margins) == 60 and min(margins) >= 0.05
