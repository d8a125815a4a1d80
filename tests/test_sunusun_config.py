"""Sunusun's configuration, plan and model folder: what runs without a GPU."""
import copy
import json
import os

import pytest
import torch

from sunusun_cases import CONFIGS, write_folder


def test_configuration_round_trip_and_plan():
    from bitnet_c_amd.config import SunusunConfig, architecture_for
    from bitnet_c_amd.config.sunusun import build_sunusun_plan
    for name, raw in CONFIGS.items():
        assert architecture_for(raw).name == "Sunusun"
        c = SunusunConfig.from_dict(raw)
        assert SunusunConfig.from_dict(c.to_dict()) == c
        plan = build_sunusun_plan(c)
        owners = [i for i, L in enumerate(raw["layers"]) if "weights_of" not in L]
        assert len(plan.layers) == len(owners) and len(plan.schedule) == len(raw["layers"])
        for i, (e, L) in enumerate(zip(plan.schedule, raw["layers"])):
            assert e.layer == owners.index(L.get("weights_of", i)) and e.kv_from is None
        t = plan.expected_tensors()
        assert t["embed"].shape == (raw["vocab"], raw["width"]) and t["head"].shape == (raw["vocab"], raw["width"])
        assert t["final.norm"].shape == ()
        for i, L in enumerate(raw["layers"]):
            p = f"l{i}."
            if "weights_of" in L:
                assert not [n for n in t if n.startswith(p)]
                continue
            assert t[p + "norm1"].shape == ()
            assert (p + "mlp.up" in t) == (L["mlp"] is not None) == (p + "norm2" in t)
            m = L["mixer"]
            if L["type"] == "wkv":
                A = m["heads"] * m["dim"]
                assert t[p + "mix.r"].shape == (A, raw["width"]) and t[p + "mix.o"].shape == (raw["width"], A)
                assert t[p + "mix.w1"].shape == (m["decay_rank"], raw["width"]) and t[p + "mix.w2"].shape == (A, m["decay_rank"])
                assert t[p + "mix.u"].shape == (m["heads"], m["dim"]) and t[p + "mix.mu.w"].shape == (raw["width"],)
            else:
                a, W = m["left"], m["right"]["width"]
                assert t[p + "mix.left.q"].shape == (a["heads"] * a["dim"], raw["width"])
                assert t[p + "mix.left.v"].shape == (a["kv_heads"] * a["vdim"], raw["width"])
                assert t[p + "mix.left.o"].shape == (raw["width"], a["heads"] * a["vdim"])
                assert t[p + "mix.left.q.norm"].shape == (a["dim"],) and t[p + "mix.left.r2"].shape == (a["heads"],)
                assert t[p + "mix.right.z"].shape == (W, raw["width"]) and t[p + "mix.right.x.b"].shape == (W,)
                assert t[p + "mix.left.out"].shape == (raw["width"],) == t[p + "mix.right.out"].shape


def test_cache_needs_a_state_per_entry_and_pages_per_attention():
    from bitnet_c_amd.cache import PagedCache
    from bitnet_c_amd.config import SunusunConfig
    from bitnet_c_amd.config.sunusun import build_sunusun_plan
    from bitnet_c_amd.parts import BLOCKS
    raw = CONFIGS["P"]
    plan = build_sunusun_plan(SunusunConfig.from_dict(raw))
    needs = [BLOCKS.build(plan.layers[e.layer].block).cache_need() for e in plan.schedule]
    for need, L in zip(needs, raw["layers"]):
        m = L["mixer"]
        if L["type"] == "wkv":
            rows = 16
            while rows < m["dim"]:
                rows *= 2                          # the kernel holds a head's rows rounded up to a power of two times 16
            assert need.kv is None and need.state.shape == (m["heads"] * rows * m["dim"] + raw["width"],)
        else:
            assert need.state.shape == (m["right"]["width"],) and need.kv.v_layout == "transposed"
            assert (need.kv.n_kv_heads, need.kv.head_dim, need.kv.v_dim) == (m["left"]["kv_heads"], m["left"]["dim"], m["left"]["vdim"])
        assert need.state.device_addressed and need.state.dtype == torch.float32
    cache = PagedCache(needs, [None] * len(needs), 256, dtype=torch.float32, device=None)
    assert len(cache.groups) == 1 and cache.groups[0].entries == [0, 3]       # the shared layer has pages of its own
    s = cache.alloc_slot()
    cache.reserve([s], [70])
    cache.commit([s], [70])
    cache.free_slot(s)
    cache.check()


def test_errors_of_a_configuration():
    from bitnet_c_amd.config import ConfigError, SunusunConfig
    ok = CONFIGS["P"]

    def broken(change):
        raw = copy.deepcopy(ok)
        change(raw)
        with pytest.raises(ConfigError):
            SunusunConfig.from_dict(raw)

    broken(lambda r: r["layers"][0].update(type="conv"))
    broken(lambda r: r["layers"][3].update(weights_of=3))
    broken(lambda r: r["layers"][3].update(weights_of=1))              # another kind of layer
    broken(lambda r: r["layers"][3]["mixer"]["right"].update(width=41))   # differs from the layer whose weights it uses
    broken(lambda r: r["layers"][1]["mixer"].pop("decay_rank"))
    broken(lambda r: r["layers"][0]["mixer"]["left"].update(kv_heads=3))
    broken(lambda r: r["layers"][2]["mlp"].update(kind="gated"))
    broken(lambda r: r.pop("norm"))
    broken(lambda r: r.update(layers=[]))


def test_a_folder_names_its_sizes_or_leaves_them_to_the_tensors(tmp_path):
    from bitnet_c_amd.config import ConfigError, load_config
    from bitnet_c_amd.weights import WeightError, open_tensors
    folder = write_folder(tmp_path / "m", CONFIGS["Q"], 1, torch.bfloat16, name_rank=False)
    raw = json.load(open(os.path.join(folder, "config.json")))
    assert all("decay_rank" not in L["mixer"] for L in raw["layers"])
    arch, cfg = load_config(folder)
    assert [L.mixer.decay_rank for L in cfg.layers if L.type == "wkv"] == [4, 4]
    plan = arch.build_plan(cfg)
    with open_tensors(folder, plan.expected_tensors()) as src:
        assert src["l1.norm1"].shape == () and src["l2.mix.w1"].shape == (4, 48)
    # a folder whose tensors do not fit its configuration is refused with every mismatch named
    raw["layers"][1]["mixer"]["right"]["width"] = 32
    json.dump(raw, open(os.path.join(folder, "config.json"), "w"))
    arch, cfg = load_config(folder)
    with pytest.raises(WeightError) as e:
        open_tensors(folder, arch.build_plan(cfg).expected_tensors())
    assert "l1.mix.right.z" in str(e.value)
    os.remove(os.path.join(folder, "model.safetensors"))
    with pytest.raises(ConfigError):
        load_config(folder)                           # no tensor gives the rank now
