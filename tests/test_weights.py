"""Safetensors reading and writing, the weight loader's error report and the
random-weights mode (no GPU).  The corrupt-file cases are the reference's
(engine/loader/safetensors_test.go:112-227)."""

import json
import os
import struct

import pytest
import torch

import tiny
from kllm_amd.config import config_from_dict, resolve_architecture
from kllm_amd.engine.model import collect_weight_specs
from kllm_amd.parts import WeightSpec
from kllm_amd.weights import (Checkpoint, SafetensorsError, WeightError, load_weights,
                              random_weights, write_random_model, write_safetensors)


def raw_file(path, header, data=b""):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        f.write(data)


def test_round_trip_with_the_library(tmp_path):
    from safetensors.torch import load_file, save_file
    t = {"a": torch.arange(12, dtype=torch.float32).reshape(3, 4),
         "b": torch.randn(5, 2).to(torch.bfloat16), "c": torch.tensor([1, 2, 3], dtype=torch.int32)}
    ours, theirs = str(tmp_path / "ours.safetensors"), str(tmp_path / "theirs.safetensors")
    write_safetensors(ours, t, metadata={"k": "v"})
    back = load_file(ours)
    save_file(t, theirs)
    with Checkpoint(theirs) as ck:
        assert ck.names() == ["a", "b", "c"]
        for name in t:
            assert torch.equal(ck.read(name), t[name]) and torch.equal(back[name], t[name])
            assert ck.entries[name].shape == tuple(t[name].shape)
    with Checkpoint(ours) as ck:
        assert ck.files[0].metadata == {"k": "v"}
        assert ck.entries["b"].dtype == "BF16" and ck.entries["b"].numel == 10


def test_corrupt_files_are_refused(tmp_path):
    p = str(tmp_path / "x.safetensors")
    with open(p, "wb") as f:
        f.write(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too short"):
        Checkpoint(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        Checkpoint(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 100) + b"{}")
    with pytest.raises(SafetensorsError, match="larger than the file"):
        Checkpoint(p)
    raw_file(p, {"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 8)
    with pytest.raises(SafetensorsError, match="outside the data"):
        Checkpoint(p)
    raw_file(p, {"t": {"dtype": "F32", "shape": [3], "data_offsets": [0, 16]}}, b"\0" * 16)
    with pytest.raises(SafetensorsError, match="need 12"):
        Checkpoint(p)
    raw_file(p, {"t": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        Checkpoint(p)
    raw_file(p, {"t": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="negative"):
        Checkpoint(p)
    raw_file(p, {"t": {"dtype": "F32", "shape": [1], "data_offsets": [4, 0]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="offsets"):
        Checkpoint(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 5) + b"[1,2]")
    with pytest.raises(SafetensorsError, match="not a JSON object"):
        Checkpoint(p)


def test_shards(tmp_path):
    write_safetensors(str(tmp_path / "m-1.safetensors"), {"a": torch.ones(2)})
    write_safetensors(str(tmp_path / "m-2.safetensors"), {"b": torch.zeros(3)})
    with Checkpoint(str(tmp_path)) as ck:            # every *.safetensors of the folder
        assert ck.names() == ["a", "b"]
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "m-1.safetensors", "b": "m-2.safetensors"}}))
    with Checkpoint(str(tmp_path)) as ck:
        assert torch.equal(ck.read("b"), torch.zeros(3))
    write_safetensors(str(tmp_path / "m-3.safetensors"), {"a": torch.ones(2)})
    os.remove(tmp_path / "model.safetensors.index.json")
    with pytest.raises(SafetensorsError, match="appears in both"):
        Checkpoint(str(tmp_path))
    with pytest.raises(SafetensorsError, match="no such file"):
        Checkpoint(str(tmp_path / "nothing"))
    (tmp_path / "empty").mkdir()
    with pytest.raises(SafetensorsError, match="no .safetensors"):
        Checkpoint(str(tmp_path / "empty"))


def llama_specs(name):
    raw = tiny.CONFIGS[name]
    return collect_weight_specs(resolve_architecture(raw).build(config_from_dict(raw)))


def test_model_wants_the_references_tensor_list():
    import plain_llama as P
    for name in ("A", "B", "C"):
        specs = {s.name: s for s in llama_specs(name)}
        shapes = P.weight_shapes(tiny.CONFIGS[name])      # backend/model.cu:873-892
        assert {k: tuple(v) for k, v in shapes.items()} == {k: s.shape for k, s in specs.items()}
        assert all(s.role == ("vector" if len(s.shape) == 1 else "matrix") for s in specs.values())
    assert "lm_head.weight" not in {s.name for s in llama_specs("B")}      # tied


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    import plain_llama as P
    cfg = tiny.CONFIGS["A"]
    w = P.random_weights(cfg, 0)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 65)
    w["model.layers.0.input_layernorm.weight"] = torch.zeros(1, 64)
    w["model.layers.7.extra.weight"] = torch.zeros(3)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)       # ignored buffer
    tiny.write_model(str(tmp_path), cfg, 0, weights=w)
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path), llama_specs("A"), torch.float32, "cpu")
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert sorted(n for n, _, _ in err.wrong_shape) == [
        "model.layers.0.input_layernorm.weight", "model.layers.0.self_attn.k_proj.weight"]
    msg = str(err)
    for word in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)",
                 "model.norm.weight", "model.layers.7.extra.weight", "[32, 65]", "[32, 64]"):
        assert word in msg


def test_dtypes_kept(tmp_path):
    import plain_llama as P
    cfg = tiny.CONFIGS["B"]
    w = P.random_weights(cfg, 1)
    tiny.write_model(str(tmp_path / "f32"), cfg, 1, "float32", weights=w)
    tiny.write_model(str(tmp_path / "bf16"), cfg, 1, "bfloat16", weights=w)
    specs = llama_specs("B")
    for store in ("f32", "bf16"):
        got = load_weights(str(tmp_path / store), specs, torch.bfloat16, "cpu")
        assert got["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
        assert got["model.norm.weight"].dtype == torch.float32          # vectors stay 32-bit
        got32 = load_weights(str(tmp_path / store), specs, torch.float32, "cpu")
        assert all(t.dtype == torch.float32 for t in got32.values())
    # a matrix stored in 32-bit is rounded to nearest even once
    a = load_weights(str(tmp_path / "f32"), specs, torch.bfloat16, "cpu")["model.embed_tokens.weight"]
    assert torch.equal(a, w["model.embed_tokens.weight"].to(torch.bfloat16))
    # a tied checkpoint may still carry lm_head.weight: named optional by the model, not read
    w2 = dict(w)
    w2["lm_head.weight"] = w["model.embed_tokens.weight"].clone()
    tiny.write_model(str(tmp_path / "tied"), cfg, 1, weights=w2)
    with pytest.raises(WeightError):
        load_weights(str(tmp_path / "tied"), specs, torch.float32, "cpu")
    load_weights(str(tmp_path / "tied"), specs, torch.float32, "cpu", optional=("lm_head.weight",))
    # integer tables stay integers, floats are refused for them
    write_safetensors(str(tmp_path / "t.safetensors"), {"idx": torch.tensor([3, 1], dtype=torch.int64)})
    t = load_weights(str(tmp_path / "t.safetensors"), [WeightSpec("idx", (2,), "table")], torch.bfloat16, "cpu")
    assert t["idx"].dtype == torch.int32 and t["idx"].tolist() == [3, 1]
    with pytest.raises(WeightError, match="wrong dtypes"):
        load_weights(str(tmp_path / "t.safetensors"), [WeightSpec("idx", (2,), "matrix")], torch.float32, "cpu")


@pytest.mark.parametrize("name,store", [("A", "float32"), ("B", "bfloat16")])
def test_random_model_folder(tmp_path, name, store):
    from safetensors.torch import load_file
    import plain_llama as P
    cfg = tiny.CONFIGS[name]
    out = write_random_model(str(tmp_path / "m"), cfg, seed=5, dtype=store)
    raw = json.loads(open(os.path.join(out, "config.json")).read())
    assert config_from_dict(raw) == config_from_dict(dict(cfg, torch_dtype=store))
    w = load_file(os.path.join(out, "model.safetensors"))
    shapes = P.weight_shapes(cfg)
    assert set(w) == set(shapes)
    for k, v in w.items():
        assert tuple(v.shape) == tuple(shapes[k]) and v.dtype == getattr(torch, store)
    emb = w["model.embed_tokens.weight"].float()
    assert abs(float(emb.std()) - 0.02) < 0.002 and abs(float(emb.mean())) < 0.002
    nw = w["model.norm.weight"].float()
    assert abs(float(nw.mean()) - 1.0) < 0.02 and 0.005 < float(nw.std()) < 0.05
    # same seed, same values, in any order and without the folder; another seed differs
    again = write_random_model(str(tmp_path / "m2"), cfg, seed=5, dtype=store)
    w2 = load_file(os.path.join(again, "model.safetensors"))
    assert all(torch.equal(w[k], w2[k]) for k in w)
    mem = random_weights(llama_specs(name), 5, getattr(torch, store))
    assert torch.equal(mem["model.layers.0.mlp.down_proj.weight"], w["model.layers.0.mlp.down_proj.weight"])
    other = random_weights(llama_specs(name), 6, getattr(torch, store))
    assert not torch.equal(other["model.embed_tokens.weight"], w["model.embed_tokens.weight"])
    # the loader reads what the writer wrote
    got = load_weights(out, llama_specs(name), torch.float32, "cpu")
    assert torch.equal(got["model.embed_tokens.weight"], emb)


KNOWN_VARIATES = [-0.207383, 0.869825, 1.187076]


def test_the_seeded_generator_depends_on_seed_name_and_index_only():
    from kllm_amd.weights.random_init import unit_variates
    z = unit_variates(3, "a.weight", 0, 200000)
    pieces = torch.cat([unit_variates(3, "a.weight", 0, 777), unit_variates(3, "a.weight", 777, 200000 - 777)])
    assert torch.equal(z, pieces)
    assert abs(float(z.mean())) < 0.01 and abs(float(z.std()) - 1.0) < 0.01 and float(z.abs().max()) < 4.9
    assert abs(float((z[:-1] * z[1:]).mean())) < 0.01                 # neighbours are uncorrelated
    other = unit_variates(3, "b.weight", 0, 200000)
    assert abs(float((z * other).mean())) < 0.01 and not torch.equal(z, other)
    assert not torch.equal(z, unit_variates(4, "a.weight", 0, 200000))
    # three known values pin the function itself (computed once with this definition)
    assert [round(float(v), 6) for v in unit_variates(1, "w", 5, 3)] == KNOWN_VARIATES
