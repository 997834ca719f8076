"""Weights by name, their errors, the safetensors container and the random-weights mode (CPU)."""
import json
import os
import struct

import pytest
import torch
from safetensors.torch import load_file as _load_file, save_file

from spyinfer_amd.config import get_architecture
from spyinfer_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, load_weights, random_tensors, write_file,
                                  write_random_model)
from tests.configs import TINY_A, TINY_B


def load_file(path):
    """Copies, so that the file may be written again while the tensors are in use."""
    return {k: v.clone() for k, v in _load_file(path).items()}


def specs_of(raw):
    arch = get_architecture("Qwen3ForCausalLM")
    return arch.build(arch.config_cls.from_dict(raw)).weight_specs()


def test_container_agrees_with_the_safetensors_library(tmp_path):
    t = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int32), "c": torch.randn(2, 2), "d": torch.randn(4).half()}
    write_file(str(tmp_path / "x.safetensors"), t)
    back = load_file(str(tmp_path / "x.safetensors"))
    assert all(torch.equal(back[k], v) for k, v in t.items())
    save_file(t, str(tmp_path / "y.safetensors"))
    f = SafetensorsFile(str(tmp_path / "y.safetensors"))
    assert all(torch.equal(f.tensor(k), v) for k, v in t.items())


def test_random_model_loads_by_name_and_is_seeded(tmp_path):
    a = write_random_model(str(tmp_path / "a"), TINY_B, seed=1)
    b = write_random_model(str(tmp_path / "b"), TINY_B, seed=1)
    c = write_random_model(str(tmp_path / "c"), TINY_B, seed=2)
    wa, wb, wc = (load_file(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert set(wa) == {s.name for s in specs_of(TINY_B)}
    assert all(torch.equal(wa[k], wb[k]) for k in wa) and not torch.equal(wa["lm_head.weight"], wc["lm_head.weight"])
    assert all(v.dtype == torch.bfloat16 for v in wa.values())
    assert json.load(open(os.path.join(a, "config.json")))["hidden_size"] == 96
    w = load_weights(a, specs_of(TINY_B), torch.bfloat16)
    assert torch.equal(w["model.norm.weight"], wa["model.norm.weight"]) and w["model.norm.weight"].dtype == torch.bfloat16
    w32 = load_weights(a, specs_of(TINY_B), torch.float32)
    assert w32["lm_head.weight"].dtype == torch.float32 and torch.equal(w32["lm_head.weight"], wa["lm_head.weight"].float())
    # streams are keyed by name: another tensor's values do not depend on the order or on what else is drawn
    sp = specs_of(TINY_B)
    assert torch.equal(random_tensors(sp[::-1], 1)["lm_head.weight"], wa["lm_head.weight"])


def test_storage_policy(tmp_path):
    """bfloat16 stays, a tensor stored in 32-bit stays 32-bit, float16 follows the run dtype."""
    folder = write_random_model(str(tmp_path / "m"), TINY_A, seed=3)
    w = load_file(os.path.join(folder, "model.safetensors"))
    w["model.norm.weight"] = w["model.norm.weight"].float()
    w["model.layers.0.mlp.up_proj.weight"] = w["model.layers.0.mlp.up_proj.weight"].half()
    write_file(os.path.join(folder, "model.safetensors"), w)
    got = load_weights(folder, specs_of(TINY_A), torch.bfloat16)
    assert got["model.norm.weight"].dtype == torch.float32
    assert got["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert got["model.layers.0.mlp.gate_proj.weight"].dtype == torch.bfloat16
    assert all(v.dtype == torch.float32 for v in load_weights(folder, specs_of(TINY_A), torch.float32).values())


def test_one_error_lists_everything(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_B, seed=4)
    w = load_file(os.path.join(folder, "model.safetensors"))
    del w["model.layers.1.self_attn.k_norm.weight"]
    del w["lm_head.weight"]
    w["model.layers.0.mlp.down_proj.weight"] = torch.zeros(96, 161, dtype=torch.bfloat16)
    w["model.layers.2.self_attn.q_proj.bias"] = torch.zeros(256, dtype=torch.bfloat16)
    w["model.norm.weight"] = torch.zeros(96, dtype=torch.int32)
    write_file(os.path.join(folder, "model.safetensors"), w)
    with pytest.raises(WeightError) as e:
        load_weights(folder, specs_of(TINY_B), torch.bfloat16)
    err = e.value
    assert sorted(err.missing) == ["lm_head.weight", "model.layers.1.self_attn.k_norm.weight"]
    assert err.unexpected == ["model.layers.2.self_attn.q_proj.bias"]
    assert [(n, list(a), list(b)) for n, a, b in err.wrong_shape] == [("model.layers.0.mlp.down_proj.weight", [96, 160], [96, 161])]
    assert err.wrong_dtype[0][0] == "model.norm.weight"
    for word in ("k_norm", "lm_head", "q_proj.bias", "[96, 161]", "missing", "unexpected", "wrong shape"):
        assert word in str(err)


def test_tied_head_stored_again_is_ignored(tmp_path):
    # src/models/qwen3.hpp:46
    folder = write_random_model(str(tmp_path / "m"), TINY_A, seed=5)
    w = load_file(os.path.join(folder, "model.safetensors"))
    w["lm_head.weight"] = torch.zeros_like(w["model.embed_tokens.weight"])
    write_file(os.path.join(folder, "model.safetensors"), w)
    got = load_weights(folder, specs_of(TINY_A), torch.bfloat16)
    assert "lm_head.weight" not in got


def test_sharded_folder(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), TINY_A, seed=6)
    w = load_file(os.path.join(folder, "model.safetensors"))
    names = sorted(w)
    half = len(names) // 2
    os.remove(os.path.join(folder, "model.safetensors"))
    write_file(os.path.join(folder, "model-00001-of-00002.safetensors"), {k: w[k] for k in names[:half]})
    write_file(os.path.join(folder, "model-00002-of-00002.safetensors"), {k: w[k] for k in names[half:]})
    wm = {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors") for i, k in enumerate(names)}
    json.dump({"weight_map": wm}, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    got = load_weights(folder, specs_of(TINY_A), torch.bfloat16)
    assert all(torch.equal(got[k], w[k]) for k in w)


def test_broken_files(tmp_path):
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        load_weights(str(tmp_path), specs_of(TINY_A), torch.bfloat16)
    p = tmp_path / "model.safetensors"
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"x": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0")
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 16"):
        SafetensorsFile(str(p))


def test_roles_of_the_random_weights_mode():
    """A vector centred on zero (a bias) has a role of its own: drawn as a norm's scale it would sit around one."""
    from spyinfer_amd.weights import WeightSpec
    specs = [WeightSpec("m", (64, 32)), WeightSpec("n", (4096,), "norm"), WeightSpec("b", (4096,), "bias"), WeightSpec("t", (9,), "table")]
    w = random_tensors(specs, 3, torch.float32, bias_std=0.05)
    assert abs(float(w["n"].mean()) - 1.0) < 0.01 and abs(float(w["b"].mean())) < 0.01 and 0.04 < float(w["b"].std()) < 0.06
    assert w["t"].dtype == torch.int32 and w["m"].shape == (64, 32)
    with pytest.raises(ValueError, match="known roles"):
        random_tensors([WeightSpec("x", (3,), "offset")], 3)


def test_every_part_of_a_model_is_named_through_its_names():
    """The position encoding's tensors lie under the prefix that the model's ``names`` give, like the other parts'."""
    from spyinfer_amd.models import DecoderModel
    from spyinfer_amd.parts import GatedMLP, LMHead, PagedAttention, PreNormBlock, RMSNorm, TokenEmbedding
    from spyinfer_amd.parts.base import PositionEncoding
    from spyinfer_amd.weights import WeightSpec

    class Table(PositionEncoding):
        def weight_specs(self, prefix):
            return [WeightSpec(prefix + ".table", (32, 64)), WeightSpec(prefix + ".offset", (64,), "bias")]

        def bind(self, prefix, weights):
            self.table, self.offset = weights[prefix + ".table"], weights[prefix + ".offset"]

    emb = TokenEmbedding(50, 64)
    block = PreNormBlock(RMSNorm(64, 1e-6), PagedAttention(64, 2, 1, 32, None), RMSNorm(64, 1e-6), GatedMLP(64, 96))
    kw = dict(config=None, embed=emb, layers=[block], final_norm=RMSNorm(64, 1e-6), lm_head=LMHead(50, 64, tied_to=emb))
    default = DecoderModel(position=Table(), **kw)
    assert {s.name for s in default.weight_specs() if "table" in s.name or "offset" in s.name} == {"model.position.table", "model.position.offset"}
    pos = Table()
    named = DecoderModel(position=pos, names=dict(position="wpe", layers="h.%d", embed="wte"), **kw)
    names = {s.name for s in named.weight_specs()}
    assert {"wpe.table", "wpe.offset", "wte.weight", "h.0.mlp.down_proj.weight", "model.norm.weight"} <= names
    assert not any(n.startswith("model.position") for n in names)
    w = random_tensors([s for s in named.weight_specs() if s.name.startswith("wpe")], 1, torch.float32)
    pos.bind("wpe", w)
    assert pos.table.shape == (32, 64) and abs(float(pos.offset.mean())) < 0.02
