"""Weights: the safetensors reader and writer, errors of the binder, the random mode (CPU)."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from sonicboom_amd.architectures.qwen2 import build_spec
from sonicboom_amd.config import Qwen2Config
from sonicboom_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, load_tensors,
                                   random_arrays, write_random_model, write_safetensors)
from sonicboom_amd.weights.safetensors_io import bf16_bits_to_f32, f32_to_bf16_bits


def test_bf16_rounding_is_nearest_even_like_torch():
    rng = np.random.default_rng(0)
    a = rng.standard_normal(4096).astype(np.float32)
    a[:6] = [0.0, -0.0, np.inf, -np.inf, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8]  # two exact ties
    ours = f32_to_bf16_bits(a)
    theirs = torch.from_numpy(a).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)
    assert np.isnan(bf16_bits_to_f32(f32_to_bf16_bits(np.array([np.nan], np.float32)))).all()


def test_folder_round_trip_and_independent_reader(model_folders, tiny_configs):
    from safetensors import safe_open
    for name, folder in model_folders.items():
        spec = build_spec(Qwen2Config.from_dict(tiny_configs[name]))
        ours = load_tensors(folder, spec, "float32", "cpu")
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            assert set(f.keys()) == {t.name for t in spec.all_tensors()}
            for k in f.keys():
                assert torch.equal(f.get_tensor(k).float(), ours[k]), k
        kept = load_tensors(folder, spec, "bfloat16", "cpu")
        assert all(t.dtype == torch.bfloat16 for t in kept.values())


def test_same_seed_same_file_other_seed_differs(tmp_path, tiny_configs):
    a, b, c = (str(tmp_path / n) for n in "abc")
    write_random_model(a, tiny_configs["A"], seed=5)
    write_random_model(b, tiny_configs["A"], seed=5)
    write_random_model(c, tiny_configs["A"], seed=6)
    ra = open(os.path.join(a, "model.safetensors"), "rb").read()
    assert ra == open(os.path.join(b, "model.safetensors"), "rb").read()
    assert ra != open(os.path.join(c, "model.safetensors"), "rb").read()


def test_random_distributions(tiny_configs):
    spec = build_spec(Qwen2Config.from_dict(tiny_configs["B"]))
    arrs = random_arrays(spec, 3)
    w = arrs["model.layers.0.mlp.up_proj.weight"]
    assert abs(w.mean()) < 2e-3 and abs(w.std() - 0.02) < 2e-3
    n = arrs["model.layers.1.input_layernorm.weight"]
    assert abs(n.mean() - 1.0) < 0.01 and abs(n.std() - 0.02) < 0.006
    b = arrs["model.layers.2.self_attn.k_proj.bias"]
    assert abs(b.mean()) < 0.02 and 0.005 < b.std() < 0.04


def test_a_tensor_stored_in_32_bit_stays_so(tmp_path, tiny_configs):
    folder = str(tmp_path / "m")
    keep = ("model.norm.weight", "model.layers.0.self_attn.q_proj.bias", "model.layers.1.mlp.down_proj.weight")
    spec = write_random_model(folder, tiny_configs["A"], seed=1, float32_tensors=keep)
    got = load_tensors(folder, spec, "bfloat16", "cpu")
    for name, t in got.items():
        assert t.dtype == (torch.float32 if name in keep else torch.bfloat16), name
    assert all(t.dtype == torch.float32 for t in load_tensors(folder, spec, "float32", "cpu").values())


def _rewrite(folder, edit):
    """Load all tensors of a folder's file raw, let ``edit`` change the dict, write it back."""
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as f:
        items = {n: (i.dtype, f.raw(n)) for n, i in f.tensors.items()}
    edit(items)
    write_safetensors(path, [(n, d, a) for n, (d, a) in items.items()])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path, tiny_configs):
    folder = str(tmp_path / "m")
    spec = write_random_model(folder, tiny_configs["B"], seed=2)

    def edit(items):
        del items["model.layers.1.self_attn.k_proj.bias"]
        del items["lm_head.weight"]
        items["model.layers.7.mlp.up_proj.weight"] = ("BF16", np.zeros((4, 4), np.uint16))
        d, a = items["model.layers.0.mlp.down_proj.weight"]
        items["model.layers.0.mlp.down_proj.weight"] = (d, a.T.copy())
        items["model.norm.weight"] = ("I32", np.zeros((96,), np.int32))
    _rewrite(folder, edit)
    with pytest.raises(WeightError) as e:
        load_tensors(folder, spec, "float32", "cpu")
    msg = str(e.value)
    assert "5 problem(s)" in msg
    assert "missing tensor: model.layers.1.self_attn.k_proj.bias" in msg
    assert "missing tensor: lm_head.weight" in msg
    assert "unexpected tensor: model.layers.7.mlp.up_proj.weight" in msg
    assert "tensor shape mismatch: model.layers.0.mlp.down_proj.weight (the file has [224, 96] BF16, the model wants [96, 224])" in msg
    assert "tensor type mismatch: model.norm.weight" in msg


def test_tied_head_tolerates_a_copy_of_the_head(tmp_path, tiny_configs):
    folder = str(tmp_path / "m")
    spec = write_random_model(folder, tiny_configs["A"], seed=2)
    assert "lm_head.weight" not in {t.name for t in spec.all_tensors()}
    _rewrite(folder, lambda items: items.__setitem__("lm_head.weight", items["model.embed_tokens.weight"]))
    got = load_tensors(folder, spec, "float32", "cpu")
    assert "lm_head.weight" not in got


def test_sharded_folder(tmp_path, tiny_configs):
    folder = str(tmp_path / "m")
    spec = write_random_model(folder, tiny_configs["A"], seed=4)
    whole = load_tensors(folder, spec, "float32", "cpu")
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as f:
        items = [(n, i.dtype, f.raw(n)) for n, i in f.tensors.items()]
    os.remove(path)
    half = len(items) // 2
    write_safetensors(os.path.join(folder, "s1.safetensors"), items[:half])
    write_safetensors(os.path.join(folder, "s2.safetensors"), items[half:])
    wm = {n: "s1.safetensors" for n, _, _ in items[:half]}
    wm.update({n: "s2.safetensors" for n, _, _ in items[half:]})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    parts = load_tensors(folder, spec, "float32", "cpu")
    assert parts.keys() == whole.keys() and all(torch.equal(parts[k], whole[k]) for k in whole)
    os.remove(os.path.join(folder, "s2.safetensors"))
    with pytest.raises(WeightError, match="io"):
        load_tensors(folder, spec, "float32", "cpu")


def test_file_errors_by_category(tmp_path):
    """Categories of /root/reference/tests/core/test_safetensors.cpp:185-321."""
    p = str(tmp_path / "x.safetensors")
    with pytest.raises(SafetensorsError, match="io"):
        SafetensorsFile(p)
    open(p, "wb").write(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(p)
    open(p, "wb").write(struct.pack("<Q", 4) + b"{{{{")
    with pytest.raises(SafetensorsError, match="format"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="truncated.*tensor t"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 12]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 16)
    with pytest.raises(SafetensorsError, match="format.*12 bytes"):
        SafetensorsFile(p)
    hdr = json.dumps({"t": {"dtype": "Q4", "shape": [4], "data_offsets": [0, 16]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 16)
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        SafetensorsFile(p)
    hdr = json.dumps({"a": {"dtype": "U8", "shape": [8], "data_offsets": [0, 8]},
                      "b": {"dtype": "U8", "shape": [8], "data_offsets": [4, 12]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 16)
    with pytest.raises(SafetensorsError, match="overlap"):
        SafetensorsFile(p)


def test_no_weights_in_folder(tmp_path, tiny_configs):
    spec = build_spec(Qwen2Config.from_dict(tiny_configs["A"]))
    with pytest.raises(WeightError, match="neither"):
        load_tensors(str(tmp_path), spec, "float32", "cpu")


def test_command_writes_a_model_folder(tmp_path, tiny_configs):
    """bin/sb-random-model: same bytes as write_random_model, an error and status 1 for a bad config."""
    import json
    import os
    import subprocess
    import sys
    from sonicboom_amd.weights import write_random_model
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(tiny_configs["B"]))
    cmd = [sys.executable, os.path.join(root, "bin", "sb-random-model")]
    r = subprocess.run(cmd + [str(cfg_path), str(tmp_path / "a"), "--seed", "11"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    write_random_model(str(tmp_path / "b"), dict(tiny_configs["B"]), seed=11)
    assert (tmp_path / "a" / "model.safetensors").read_bytes() == (tmp_path / "b" / "model.safetensors").read_bytes()
    bad = dict(tiny_configs["B"])
    del bad["hidden_size"]
    cfg_path.write_text(json.dumps(bad))
    r = subprocess.run(cmd + [str(cfg_path), str(tmp_path / "c")], capture_output=True, text=True)
    assert r.returncode == 1 and "hidden_size" in r.stderr


def test_tensors_are_read_as_they_are_asked_for(model_folders, tiny_configs):
    """open_tensors checks everything first, then reads a tensor when a part asks for it and
    forgets it when the model pops it; the values are load_tensors' own."""
    from sonicboom_amd.weights import open_tensors, random_source
    folder = model_folders["B"]
    spec = build_spec(Qwen2Config.from_dict(tiny_configs["B"]))
    whole = load_tensors(folder, spec, "bfloat16", "cpu")
    src = open_tensors(folder, spec, "bfloat16", "cpu")
    assert src.keys() == sorted(whole) and not src._kept
    name = "model.layers.1.mlp.down_proj.weight"
    assert name in src and "no.such.tensor" not in src and src.get("no.such.tensor") is None
    t = src.get(name)
    assert torch.equal(t, whole[name]) and src.get(name) is t and list(src._kept) == [name]
    assert src.pop(name) is t and name not in src and src.pop(name, None) is None
    with pytest.raises(KeyError):
        src["model.layers.9.mlp.down_proj.weight"]
    src.close()
    # drawn on demand: any order of asking gives the same values
    a, b = random_source(spec, 3, "float32", "cpu"), random_source(spec, 3, "float32", "cpu")
    names = a.keys()
    for n in names:
        a.get(n)
    for n in reversed(names):
        b.get(n)
    assert all(torch.equal(a.get(n), b.get(n)) for n in names)
    assert not torch.equal(a.get(names[0]), random_source(spec, 4, "float32", "cpu").get(names[0]))
