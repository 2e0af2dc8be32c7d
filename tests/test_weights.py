"""Weights: the folder format, the loader's one error, random folders."""
import json
import os

import pytest
import torch

from trapetum_amd.config import Gemma2Config
from trapetum_amd.weights import (SafeTensorsFile, WeightError, WeightFileError, WeightFolder, write_model_folder,
                                  write_safetensors)

from .cpu_engine import load_cpu_model
from .tiny import TINY_A, TINY_A_INIT, make_folder


def rewrite(folder, change):
    src = WeightFolder(folder)
    tensors = {n: src.tensor(n).clone() for n in src.names()}
    src.close()
    change(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)


def test_random_folder_is_reproducible_and_bf16(tmp_path):
    a = make_folder(tmp_path / "x", "A")
    b = make_folder(tmp_path / "y", "A")
    fa, fb = WeightFolder(a), WeightFolder(b)
    assert sorted(fa.names()) == sorted(fb.names()) and len(fa.names()) == 2 + 11 * 2
    for n in fa.names():
        assert fa.dtype(n) == torch.bfloat16 and torch.equal(fa.tensor(n), fb.tensor(n))
    assert "lm_head.weight" not in fa                                   # tied: the head is the embedding
    w = fa.tensor("model.layers.1.mlp.down_proj.weight").float()
    assert tuple(w.shape) == (64, 128) and abs(float(w.std()) - 0.02) < 0.002
    n = fa.tensor("model.layers.0.input_layernorm.weight").float()
    assert abs(float(n.std()) - 0.1) < 0.04
    other = write_model_folder(Gemma2Config.from_kwargs(**TINY_A), str(tmp_path / "z"), seed=1)
    assert not torch.equal(WeightFolder(other).tensor("model.norm.weight"), fa.tensor("model.norm.weight"))
    assert json.load(open(os.path.join(a, "config.json")))["architectures"] == ["Gemma2ForCausalLM"]


def test_one_error_lists_everything(tmp_path):
    folder = make_folder(tmp_path, "A")

    def change(t):
        del t["model.layers.0.self_attn.k_proj.weight"]
        del t["model.norm.weight"]
        t["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)
        t["model.layers.1.mlp.up_proj.weight"] = torch.zeros(64, 128, dtype=torch.bfloat16)
        t["model.layers.1.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    rewrite(folder, change)
    with pytest.raises(WeightError) as e:
        load_cpu_model(folder)
    err = e.value
    assert err.missing == ["model.layers.0.self_attn.k_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["lm_head.weight"]
    assert err.wrong_shape == [("model.layers.1.mlp.up_proj.weight", (128, 64), (64, 128))]
    assert [n for n, _, _ in err.wrong_dtype] == ["model.layers.1.input_layernorm.weight"]
    text = str(err)
    for piece in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (1)", "expected [128, 64], found [64, 128]"):
        assert piece in text


def test_stored_width_is_kept(tmp_path):
    folder = make_folder(tmp_path, "A")
    rewrite(folder, lambda t: t.update({"model.norm.weight": t["model.norm.weight"].float() + 1e-4}))
    model, _ = load_cpu_model(folder)
    # a tensor stored in 32 bits stays so: the norm's gain sees the 1e-4 that bf16 would have rounded away
    src = WeightFolder(folder)
    want = src.tensor("model.norm.weight").float() + 1.0
    assert src.dtype("model.norm.weight") == torch.float32 and torch.equal(model.final_norm.gain, want)


def test_malformed_files(tmp_path):
    folder = make_folder(tmp_path, "A")
    path = os.path.join(folder, "model.safetensors")
    raw = open(path, "rb").read()
    open(path, "wb").write(raw[:len(raw) // 2])
    with pytest.raises(WeightFileError, match="needs .* bytes"):
        SafeTensorsFile(path)
    open(path, "wb").write(b"\x05\x00")
    with pytest.raises(WeightFileError, match="too short"):
        SafeTensorsFile(path)
    open(path, "wb").write((10 ** 9).to_bytes(8, "little") + b"{}")
    with pytest.raises(WeightFileError, match="runs past the end"):
        SafeTensorsFile(path)
    os.remove(path)
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        WeightFolder(folder)


def test_sharded_folder(tmp_path):
    folder = make_folder(tmp_path, "A")
    src = WeightFolder(folder)
    names = sorted(src.names())
    half = len(names) // 2
    write_safetensors(os.path.join(folder, "s1.safetensors"), {n: src.tensor(n).clone() for n in names[:half]})
    write_safetensors(os.path.join(folder, "s2.safetensors"), {n: src.tensor(n).clone() for n in names[half:]})
    ref, _ = load_cpu_model(folder)
    src.close()
    os.remove(os.path.join(folder, "model.safetensors"))
    index = {"weight_map": {n: ("s1.safetensors" if i < half else "s2.safetensors") for i, n in enumerate(names)}}
    json.dump(index, open(os.path.join(folder, "model.safetensors.index.json"), "w"))
    model, _ = load_cpu_model(folder)
    assert torch.equal(model.head.weight, ref.head.weight) and torch.equal(model.layers[1].block.mixer.w_o, ref.layers[1].block.mixer.w_o)
