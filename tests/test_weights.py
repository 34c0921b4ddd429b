"""Loading by tensor name: packing, types, tied head, and the one error that lists
everything missing, unexpected and mis-shaped."""

import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from atom_amd.config import build_model, model_config_from_dict
from atom_amd.weights import (DictSource, WeightError, expected_tensors, load_model_folder, load_weights,
                              random_state_dict, write_random_model)
from helpers import tiny_folder
from tiny import TINY_A, TINY_B, TINY_C


def test_random_folder_has_the_checkpoint_names(tmp_path):
    cfg = model_config_from_dict(TINY_C)
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=3)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    assert tensors["model.layers.3.self_attn.q_proj.weight"].shape == (8 * 64, 136)
    assert tensors["model.layers.0.self_attn.k_proj.bias"].shape == (2 * 64,)
    assert tensors["model.layers.1.mlp.gate_proj.weight"].shape == (200, 136)
    assert tensors["model.layers.2.self_attn.q_norm.weight"].shape == (64,)
    assert tensors["lm_head.weight"].shape == (517, 136) and tensors["model.norm.weight"].dtype == torch.bfloat16
    assert "lm_head.weight" not in random_state_dict(model_config_from_dict(TINY_A), 0)
    # seeded: same seed same values, another seed other values; norm weights sit around one
    again = random_state_dict(cfg, 3)
    assert all(torch.equal(tensors[k], again[k]) for k in tensors)
    other = random_state_dict(cfg, 4)
    assert not torch.equal(other["lm_head.weight"], again["lm_head.weight"])
    assert abs(float(again["model.norm.weight"].float().mean()) - 1.0) < 0.1
    assert float(again["model.norm.weight"].float().std()) > 0.02


def test_packed_rows_and_types():
    cfg = model_config_from_dict(TINY_B)
    state = random_state_dict(cfg, 1, dtype=torch.bfloat16)
    model = build_model(cfg)
    load_weights(model, DictSource(state), "cpu", torch.bfloat16)
    attn = model.blocks[1].mixer
    qkv = attn.params["qkv.weight"]
    assert qkv.shape == ((6 + 2 * 3) * 32, 96) and qkv.dtype == torch.bfloat16
    p = "model.layers.1.self_attn."
    assert torch.equal(qkv[:192], state[p + "q_proj.weight"])           # rows q | k | v
    assert torch.equal(qkv[192:288], state[p + "k_proj.weight"])
    assert torch.equal(qkv[288:], state[p + "v_proj.weight"])
    gu = model.blocks[1].ffn.params["gate_up.weight"]
    assert torch.equal(gu[:160], state["model.layers.1.mlp.gate_proj.weight"])   # gate first
    assert torch.equal(gu[160:], state["model.layers.1.mlp.up_proj.weight"])
    assert attn.params["q_norm.weight"].dtype == torch.float32           # norm weights are float32
    assert model.final_norm.params["weight"].dtype == torch.float32
    # 32-bit path: everything widened, exactly
    model32 = build_model(cfg)
    load_weights(model32, DictSource(state), "cpu", torch.float32)
    assert model32.blocks[1].mixer.params["qkv.weight"].dtype == torch.float32
    assert torch.equal(model32.blocks[1].mixer.params["qkv.weight"], qkv.float())


def test_tensor_stored_in_32_bit_stays_so():
    cfg = model_config_from_dict(TINY_A)
    state = random_state_dict(cfg, 0, dtype=torch.float32)
    model = build_model(cfg)
    load_weights(model, DictSource(state), "cpu", torch.bfloat16)
    assert model.embedding.params["weight"].dtype == torch.float32
    assert torch.equal(model.embedding.params["weight"], state["model.embed_tokens.weight"])
    half = {k: v.half() for k, v in state.items()}
    model16 = build_model(cfg)
    load_weights(model16, DictSource(half), "cpu", torch.bfloat16)
    assert model16.embedding.params["weight"].dtype == torch.bfloat16


def test_tied_head_shares_the_embedding(tmp_path):
    cfg = model_config_from_dict(TINY_A)
    model = build_model(cfg)
    load_model_folder(model, tiny_folder("A"), "cpu", torch.bfloat16)
    assert model.head.weight is model.embedding.params["weight"]
    # a tied checkpoint that still carries lm_head.weight loads too
    state = random_state_dict(cfg, 0)
    state["lm_head.weight"] = state["model.embed_tokens.weight"].clone()
    load_weights(build_model(cfg), DictSource(state), "cpu", torch.bfloat16)


def test_one_error_lists_missing_unexpected_and_misshaped():
    cfg = model_config_from_dict(TINY_B)
    state = random_state_dict(cfg, 1)
    del state["model.layers.0.mlp.up_proj.weight"]
    del state["model.norm.weight"]
    state["model.layers.0.self_attn.gate.weight"] = torch.zeros(16)
    state["model.layers.2.self_attn.o_proj.weight"] = torch.zeros(192, 96)     # transposed
    state["model.layers.1.self_attn.k_norm.weight"] = torch.zeros(31)
    with pytest.raises(WeightError) as e:
        load_weights(build_model(cfg), DictSource(state, "test"), "cpu", torch.bfloat16)
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.gate.weight"]
    assert [m[0] for m in err.mismatched] == ["model.layers.1.self_attn.k_norm.weight",
                                              "model.layers.2.self_attn.o_proj.weight"]
    text = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (2)", "(192, 96)", "(96, 192)", "up_proj"):
        assert needle in text


def test_names_the_reference_drops_are_dropped(caplog):
    """atom/model_loader/weight_names.py:160-201: ``*kv_scale``, ``*inv_freq*`` and layers beyond the
    model's last are left aside without an error; a name that only looks similar is still an error."""
    import logging
    cfg = model_config_from_dict(TINY_B)
    state = random_state_dict(cfg, 1)
    state["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    state["model.layers.1.self_attn.k_proj.kv_scale"] = torch.ones(1)
    state[f"model.layers.{cfg.num_hidden_layers}.mlp.up_proj.weight"] = torch.zeros(3, 3)
    state[f"model.layers.{cfg.num_hidden_layers + 7}.anything"] = torch.zeros(2)
    with caplog.at_level(logging.DEBUG, logger="atom_amd"):
        model = build_model(cfg)
        load_weights(model, DictSource(state), "cpu", torch.bfloat16)
    dropped = [r.getMessage() for r in caplog.records if "dropped" in r.getMessage()]
    assert len(dropped) == 4 and any("inv_freq" in d for d in dropped)
    state["model.layers.0.self_attn.kv_scales"] = torch.ones(1)      # neither suffix nor substring
    state["model.layers.x.mlp.up_proj.weight"] = torch.ones(1)       # no layer number
    with pytest.raises(WeightError) as e:
        load_weights(build_model(cfg), DictSource(state), "cpu", torch.bfloat16)
    assert e.value.unexpected == ["model.layers.0.self_attn.kv_scales", "model.layers.x.mlp.up_proj.weight"]
    assert not e.value.missing and not e.value.mismatched


def test_a_checkpoint_runs_with_fewer_layers_than_it_holds(tmp_path):
    """The reference's truncation path: ``--hf-overrides '{"num_hidden_layers": N}'`` (atom/config.py:1699-1701)
    with the tensors of the layers past N dropped by name (weight_names.py:197-201)."""
    from atom_amd.config import Config
    folder = tiny_folder("B")                      # three layers
    full = Config(model=folder, dtype="fp32")
    cut = Config(model=folder, dtype="fp32", hf_overrides={"num_hidden_layers": 2})
    assert full.model_config.num_hidden_layers == 3 and cut.model_config.num_hidden_layers == 2
    small, whole = build_model(cut.model_config), build_model(full.model_config)
    load_model_folder(small, folder, "cpu", torch.float32)
    load_model_folder(whole, folder, "cpu", torch.float32)
    assert len(small.blocks) == 2
    for a, b in zip(small.blocks, whole.blocks):
        for pa, pb in zip(a.walk(), b.walk()):
            for name in pa.params:
                assert torch.equal(pa.params[name], pb.params[name])
    # more layers than the checkpoint holds is still an error that names what is missing
    more = Config(model=folder, dtype="fp32", hf_overrides={"num_hidden_layers": 4})
    with pytest.raises(WeightError, match=r"model\.layers\.3\."):
        load_model_folder(build_model(more.model_config), folder, "cpu", torch.float32)


def test_untied_model_needs_its_head():
    cfg = model_config_from_dict(TINY_B)
    state = random_state_dict(cfg, 1)
    del state["lm_head.weight"]
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_weights(build_model(cfg), DictSource(state), "cpu", torch.bfloat16)


def test_sharded_folder_and_missing_shard(tmp_path):
    import json
    cfg = model_config_from_dict(TINY_A)
    state = random_state_dict(cfg, 0)
    names = sorted(state)
    half = len(names) // 2
    folder = tmp_path / "sharded"
    folder.mkdir()
    cfg.save(str(folder))
    save_file({k: state[k] for k in names[:half]}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({k: state[k] for k in names[half:]}, str(folder / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, k in enumerate(names)}}
    (folder / "model.safetensors.index.json").write_text(json.dumps(index))
    load_model_folder(build_model(cfg), str(folder), "cpu", torch.bfloat16)
    os.remove(folder / "model-00002-of-00002.safetensors")
    with pytest.raises(FileNotFoundError, match="model-00002-of-00002"):
        load_model_folder(build_model(cfg), str(folder), "cpu", torch.bfloat16)


def test_expected_names_cover_the_checkpoint():
    cfg = model_config_from_dict(TINY_C)
    names = set(expected_tensors(build_model(cfg)))
    assert names == set(random_state_dict(cfg, 5))
    assert len(names) == 4 * (3 + 3 + 1 + 2 + 2 + 3) + 3
