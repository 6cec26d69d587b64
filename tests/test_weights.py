"""Weights by name: round trip, the one error that lists everything, dtypes (no GPU)."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from dryft_amd.engine.model import DecoderModel
from dryft_amd.models import resolve_architecture
from dryft_amd.weights import (INT_TABLE, MATRIX, VECTOR, ShardSet, TensorSpec, WeightError, load_tensors,
                               random_tensors, write_model_dir)
from helpers import TINY_A, TINY_B, make_model_dir


def model_for(raw, dtype=torch.float32):
    arch = resolve_architecture(raw)
    return DecoderModel(arch.plan(arch.config_class.from_dict(raw)), dtype, "cpu")


def test_random_folder_reads_back_equal(tmp_path):
    path = make_model_dir(str(tmp_path / "m"), TINY_B, seed=3, norm_std=0.1)
    assert sorted(os.listdir(path)) == ["config.json", "model.safetensors"]
    model = model_for(TINY_B)
    specs = model.tensor_specs()
    again = random_tensors(specs, 3, torch.bfloat16, norm_std=0.1)
    loaded = load_tensors(path, specs, torch.bfloat16)
    assert set(loaded) == {s.name for s in specs}
    for s in specs:
        assert loaded[s.name].dtype == torch.bfloat16 and tuple(loaded[s.name].shape) == s.shape
        assert torch.equal(loaded[s.name], again[s.name]), s.name
    other = random_tensors(specs, 4, torch.bfloat16, norm_std=0.1)
    assert not torch.equal(other[specs[0].name], again[specs[0].name])
    norm = loaded["model.layers.0.input_layernorm.weight"].float()
    assert 0.05 < float(norm.std()) < 0.2 and abs(float(norm.mean()) - 1) < 0.05
    emb = loaded["model.embed_tokens.weight"].float()
    assert 0.015 < float(emb.std()) < 0.025
    # norm weights are exactly one when no spread is asked for
    ones = random_tensors(specs, 3, torch.bfloat16)["model.norm.weight"]
    assert torch.equal(ones, torch.ones_like(ones))


def test_float32_mode_widens_exactly(tmp_path):
    path = make_model_dir(str(tmp_path / "m"), TINY_A, seed=1)
    specs = model_for(TINY_A).tensor_specs()
    low = load_tensors(path, specs, torch.bfloat16)
    wide = load_tensors(path, specs, torch.float32)
    for name, t in wide.items():
        assert t.dtype == torch.float32 and torch.equal(t, low[name].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    path = make_model_dir(str(tmp_path / "m"), TINY_B, seed=3)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.weight"] = t["model.layers.0.self_attn.q_proj.weight"][:, :-1].contiguous()
    t["model.layers.2.self_attn.k_norm.weight"] = torch.ones(7, dtype=torch.bfloat16)
    t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(4)
    t["extra.weight"] = torch.ones(2, 2)
    save_file(t, file)
    with pytest.raises(WeightError) as e:
        load_tensors(path, model_for(TINY_B).tensor_specs(), torch.bfloat16)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["extra.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert [w[0] for w in err.wrong_shape] == ["model.layers.0.self_attn.q_proj.weight",
                                               "model.layers.2.self_attn.k_norm.weight"]
    assert err.wrong_shape[0][1:] == ((256, 96), (256, 95))
    text = str(err)
    for name in err.missing + err.unexpected + [w[0] for w in err.wrong_shape]:
        assert name in text


def test_untied_model_needs_its_head_and_tied_copy_must_match(tmp_path):
    path = make_model_dir(str(tmp_path / "b"), TINY_B, seed=3)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    del t["lm_head.weight"]
    save_file(t, file)
    with pytest.raises(WeightError) as e:
        load_tensors(path, model_for(TINY_B).tensor_specs(), torch.bfloat16)
    assert e.value.missing == ["lm_head.weight"]
    # tied: a copy of the embedding may be present, and must equal it (reference weights.py:82-88)
    path = make_model_dir(str(tmp_path / "a"), TINY_A, seed=3)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    save_file(t, file)
    model = model_for(TINY_A)
    tensors = load_tensors(path, model.tensor_specs(), torch.float32, ignore=model.optional_names())
    model.load(tensors)
    assert model.head.weight is model.embedding.weight
    t["lm_head.weight"] = t["lm_head.weight"] + 1
    save_file(t, file)
    model = model_for(TINY_A)
    with pytest.raises(ValueError, match="differs from model.embed_tokens.weight"):
        model.load(load_tensors(path, model.tensor_specs(), torch.float32, ignore=model.optional_names()))


def test_dtype_rule(tmp_path):
    """bfloat16 by default; a vector stored in 32-bit stays 32-bit; integer tables become int32."""
    tensors = {"m": torch.randn(4, 6), "m16": torch.randn(4, 6).to(torch.float16), "v32": torch.randn(6),
               "vb": torch.randn(6).to(torch.bfloat16), "ids": torch.arange(5, dtype=torch.int64)}
    write_model_dir(str(tmp_path), {"architectures": ["none"]}, tensors)
    specs = [TensorSpec("m", (4, 6), MATRIX), TensorSpec("m16", (4, 6), MATRIX), TensorSpec("v32", (6,), VECTOR),
             TensorSpec("vb", (6,), VECTOR), TensorSpec("ids", (5,), INT_TABLE)]
    got = load_tensors(str(tmp_path), specs, torch.bfloat16)
    assert [got[n].dtype for n in ("m", "m16", "v32", "vb", "ids")] == \
        [torch.bfloat16, torch.bfloat16, torch.float32, torch.bfloat16, torch.int32]
    assert torch.equal(got["v32"], tensors["v32"]) and got["ids"].tolist() == [0, 1, 2, 3, 4]
    wide = load_tensors(str(tmp_path), specs, torch.float32)
    assert [wide[n].dtype for n in ("m", "m16", "v32", "vb", "ids")] == [torch.float32] * 4 + [torch.int32]
    with pytest.raises(WeightError, match="integer table stored as"):
        load_tensors(str(tmp_path), [TensorSpec("m", (4, 6), INT_TABLE)] + specs[1:], torch.bfloat16)


def test_shards_are_found_through_the_index(tmp_path):
    path = make_model_dir(str(tmp_path / "m"), TINY_A, seed=9)
    file = os.path.join(path, "model.safetensors")
    t = load_file(file)
    names = sorted(t)
    half = len(names) // 2
    save_file({n: t[n] for n in names[:half]}, os.path.join(path, "model-00001-of-00002.safetensors"))
    save_file({n: t[n] for n in names[half:]}, os.path.join(path, "model-00002-of-00002.safetensors"))
    os.remove(file)
    index = {"weight_map": {n: f"model-0000{1 if i < half else 2}-of-00002.safetensors" for i, n in enumerate(names)}}
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    got = load_tensors(path, model_for(TINY_A).tensor_specs(), torch.bfloat16)
    assert all(torch.equal(got[n], t[n]) for n in names)
    # the index alone says where a tensor lives: a file of the folder that it does not name is never opened,
    # and a tensor that the named shard lacks is reported as missing
    with open(os.path.join(path, "stray.safetensors"), "w") as f:
        f.write("not a safetensors file")
    assert ShardSet(path).files() == [os.path.join(path, f"model-0000{i}-of-00002.safetensors") for i in (1, 2)]
    load_tensors(path, model_for(TINY_A).tensor_specs(), torch.bfloat16)
    index["weight_map"][names[0]] = "model-00002-of-00002.safetensors"
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    with pytest.raises(WeightError) as e:
        load_tensors(path, model_for(TINY_A).tensor_specs(), torch.bfloat16)
    assert e.value.missing == [names[0]]
    with pytest.raises(FileNotFoundError):
        load_tensors(str(tmp_path / "empty"), [], torch.bfloat16)


def test_fused_rows_equal_their_parts(tmp_path):
    """q;k;v and gate;up are stacked by rows (reference weights.py:93-100)."""
    path = make_model_dir(str(tmp_path / "m"), TINY_B, seed=3)
    model = model_for(TINY_B)
    tensors = load_tensors(path, model.tensor_specs(), torch.float32)
    handed = dict(tensors)
    model.load(handed)
    assert not handed, "loading hands every tensor on and keeps none in the dictionary it was given"
    att, ffn = model.blocks[1].mixer, model.blocks[1].ffn
    p = "model.layers.1."
    assert torch.equal(att.w_qkv[:256], tensors[p + "self_attn.q_proj.weight"])
    assert torch.equal(att.w_qkv[256:320], tensors[p + "self_attn.k_proj.weight"])
    assert torch.equal(att.w_qkv[320:], tensors[p + "self_attn.v_proj.weight"])
    assert torch.equal(ffn.w_gate_up[:224], tensors[p + "mlp.gate_proj.weight"])
    assert torch.equal(ffn.w_gate_up[224:], tensors[p + "mlp.up_proj.weight"])


def test_command_line_make_model_round_trip(tmp_path):
    """`python -m dryft_amd make-model` writes the folder that the random-weights mode describes: the same
    configuration and, tensor for tensor, what the seed gives."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "made")
    proc = subprocess.run([sys.executable, "-m", "dryft_amd", "make-model", "--preset", "tiny-b", "--weight-seed", "3",
                           "--norm-std", "0.1", "--out", out], capture_output=True, text=True, cwd=root, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.strip() == out
    with open(os.path.join(out, "config.json")) as f:
        raw = json.load(f)
    from dryft_amd.models import load_preset
    assert raw == load_preset("tiny-b")
    model = model_for(raw)
    specs = model.tensor_specs()
    loaded = load_tensors(out, specs, torch.bfloat16)
    want = random_tensors(specs, 3, torch.bfloat16, norm_std=0.1)
    assert all(torch.equal(loaded[s.name], want[s.name]) for s in specs)
    # a config.json of one's own instead of a preset, in float32
    cfg_path = str(tmp_path / "c.json")
    with open(cfg_path, "w") as f:
        json.dump(dict(TINY_A, vocab_size=300), f)
    out2 = str(tmp_path / "made2")
    proc = subprocess.run([sys.executable, "-m", "dryft_amd", "make-model", "--config", cfg_path, "--dtype", "fp32",
                           "--out", out2], capture_output=True, text=True, cwd=root, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    t = load_file(os.path.join(out2, "model.safetensors"))
    assert t["model.embed_tokens.weight"].shape == (300, 64) and t["model.embed_tokens.weight"].dtype == torch.float32
    assert "lm_head.weight" not in t
