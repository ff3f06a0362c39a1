"""The safetensors reader, the by-name loader's one error, tied heads, random weights (no GPU:
parameters are placed on the CPU device, which the loader treats like any other)."""
import json
import os
import struct

import pytest
import torch

from llmengine.config import parse_config
from llmengine.models.llama import build_llama
from llmengine.parts.base import Placement
from llmengine.weights import (SafetensorsError, TensorIndex, WeightError, load_model_weights, random_state,
                               write_random_model, write_state_dict)
from tiny_models import A_INIT, B_INIT, TINY_A, TINY_B, make_model_dir

CPU32 = Placement(torch.device("cpu"), torch.float32)
CPU16 = Placement(torch.device("cpu"), torch.bfloat16)


def _state(cfg, seed=0, dtype=torch.float32):
    return dict(random_state(cfg, seed, dtype))


def _write(tmp_path, cfg, tensors):
    os.makedirs(tmp_path, exist_ok=True)
    with open(os.path.join(tmp_path, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_state_dict(os.path.join(tmp_path, "model.safetensors"), tensors)
    return str(tmp_path)


def test_round_trip_against_the_library(tmp_path):
    from safetensors.torch import load_file, save_file
    d = make_model_dir(tmp_path / "m", TINY_B, B_INIT, torch.bfloat16)
    lib = load_file(os.path.join(d, "model.safetensors"))           # our writer, their reader
    ours = TensorIndex(d)
    assert sorted(lib) == ours.names()
    for k, v in lib.items():
        assert torch.equal(v, ours.read(k))
    save_file({k: v.clone() for k, v in lib.items()}, str(tmp_path / "m" / "model.safetensors"))
    theirs = TensorIndex(d)                                         # their writer, our reader
    for k, v in lib.items():
        assert torch.equal(v, theirs.read(k))


def test_random_weights_are_reproducible_and_as_specified(tmp_path):
    a = _state(TINY_B, 1)
    b = _state(TINY_B, 1)
    c = _state(TINY_B, 2)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    s = dict(random_state(TINY_B, 1, torch.float32, 0.05, 1.0, 0.1))
    assert abs(s["model.layers.0.mlp.up_proj.weight"].std().item() - 0.05) < 5e-3
    assert abs(s["model.norm.weight"].mean().item() - 1.0) < 0.05
    assert 0.05 < s["model.norm.weight"].std().item() < 0.2
    ones = dict(random_state(TINY_A, 0, torch.float32, 0.02, 1.0, 0.0))
    assert torch.all(ones["model.layers.1.input_layernorm.weight"] == 1.0)
    assert "lm_head.weight" not in ones and "lm_head.weight" in s            # tied A has no head tensor
    d = write_random_model(TINY_A, str(tmp_path / "a"), 0, torch.bfloat16)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(d, "config.json")))["hidden_size"] == 64


def test_names_shapes_and_fusing(tmp_path):
    cfg = parse_config(TINY_B)
    model = build_llama(cfg)
    specs = model.named_specs()
    assert specs["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)
    assert specs["model.layers.0.mlp.down_proj.weight"].shape == (96, 256)
    assert specs["lm_head.weight"].shape == (384, 96)
    d = _write(tmp_path / "b", TINY_B, _state(TINY_B, 1))
    load_model_weights(model, d, CPU32)
    w = _state(TINY_B, 1)
    attn = model.layers[1].mixer
    want = torch.cat([w[f"model.layers.1.self_attn.{n}_proj.weight"] for n in "qkv"])
    assert torch.equal(attn.w_qkv, want)
    mlp = model.layers[1].feed_forward
    g = mlp.group
    fused = mlp.w_gate_up.view(-1, 2, g, 96)
    assert torch.equal(fused[:, 0].reshape(-1, 96), w["model.layers.1.mlp.gate_proj.weight"])
    assert torch.equal(fused[:, 1].reshape(-1, 96), w["model.layers.1.mlp.up_proj.weight"])


def test_storage_types(tmp_path):
    bf = _write(tmp_path / "bf", TINY_A, _state(TINY_A, 0, torch.bfloat16))
    m = build_llama(parse_config(TINY_A))
    load_model_weights(m, bf, CPU16)
    assert m.embedding.weight.dtype == torch.bfloat16 and m.layers[0].mixer.w_qkv.dtype == torch.bfloat16
    m32 = build_llama(parse_config(TINY_A))
    load_model_weights(m32, bf, CPU32)
    assert m32.embedding.weight.dtype == torch.float32
    from llmengine import ops
    assert ops.is_blocked(m.embedding.weight) and not ops.is_blocked(m32.embedding.weight)   # bfloat16 matrices: blocked
    assert torch.equal(m32.embedding.weight, ops.unblock_weight(m.embedding.weight).float())   # widening is exact
    # a tensor stored in 32-bit stays so in the bfloat16 model
    mixed = _state(TINY_A, 0, torch.bfloat16)
    mixed["model.norm.weight"] = mixed["model.norm.weight"].float()
    mx = build_llama(parse_config(TINY_A))
    load_model_weights(mx, _write(tmp_path / "mx", TINY_A, mixed), CPU16)
    assert mx.final_norm.weight.dtype == torch.float32 and mx.layers[0].mixer_norm.weight.dtype == torch.bfloat16


def test_tied_head_is_the_embedding(tmp_path):
    tied = build_llama(parse_config(TINY_A))
    load_model_weights(tied, _write(tmp_path / "a", TINY_A, _state(TINY_A)), CPU32)
    assert tied.head.weight.data_ptr() == tied.embedding.weight.data_ptr()
    # a tied checkpoint that also stores lm_head.weight: accepted, the embedding is used
    both = _state(TINY_A)
    both["lm_head.weight"] = torch.zeros(256, 64)
    t2 = build_llama(parse_config(TINY_A))
    load_model_weights(t2, _write(tmp_path / "a2", TINY_A, both), CPU32)
    assert t2.head.weight.data_ptr() == t2.embedding.weight.data_ptr()
    # .. unless it disagrees with the embedding in shape or type (src/weights.cpp:259-264)
    for bad, what in ((torch.zeros(64, 256), "[64,256]"), (torch.zeros(255, 64), "[255,64]"),
                      (torch.zeros(256, 64, dtype=torch.bfloat16), "bfloat16")):
        state = _state(TINY_A)
        state["lm_head.weight"] = bad
        with pytest.raises(WeightError) as e:
            load_model_weights(build_llama(parse_config(TINY_A)), _write(tmp_path / f"bad{what}", TINY_A, state), CPU32)
        assert ("tie_word_embeddings=true but lm_head.weight shape/dtype disagrees with model.embed_tokens.weight"
                in str(e.value)) and what in str(e.value)
        assert e.value.wrong_shape == ["lm_head.weight"] and not e.value.missing and not e.value.unexpected
    untied = build_llama(parse_config(TINY_B))
    load_model_weights(untied, _write(tmp_path / "b", TINY_B, _state(TINY_B)), CPU32)
    assert untied.head.weight.data_ptr() != untied.embedding.weight.data_ptr()


def test_one_error_lists_everything(tmp_path):
    w = _state(TINY_B)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.k_proj.weight"] = w["model.layers.0.self_attn.k_proj.weight"].T.contiguous()
    w["model.layers.9.extra.weight"] = torch.zeros(2, 2)
    with pytest.raises(WeightError) as e:
        load_model_weights(build_llama(parse_config(TINY_B)), _write(tmp_path / "bad", TINY_B, w), CPU32)
    msg = str(e.value)
    assert "missing weight: model.layers.1.mlp.up_proj.weight" in msg
    assert "missing weight: model.norm.weight" in msg
    assert "shape mismatch for model.layers.0.self_attn.k_proj.weight: expected [32,96], got [96,32]" in msg
    assert "unexpected tensor: model.layers.9.extra.weight" in msg
    assert e.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.value.unexpected == ["model.layers.9.extra.weight"]
    assert e.value.wrong_shape == ["model.layers.0.self_attn.k_proj.weight"]


def _raw_file(path, header: dict, data: bytes):
    blob = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)) + blob + data)


@pytest.mark.parametrize("header,data,needle", [
    ({"t": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 12]}}, b"\0" * 16, "byte-count mismatch"),
    ({"t": {"dtype": "F32", "shape": [-1, 2], "data_offsets": [0, 8]}}, b"\0" * 8, "negative shape dim"),
    ({"t": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 64]}}, b"\0" * 16, "offsets out of range"),
    ({"t": {"dtype": "F64", "shape": [1], "data_offsets": [0, 8]}}, b"\0" * 8, "unsupported safetensors dtype"),
    ({"t": {"dtype": "F32", "shape": [1 << 40, 1 << 40], "data_offsets": [0, 8]}}, b"\0" * 8, "overflow"),
])
def test_malformed_files(tmp_path, header, data, needle):
    _raw_file(tmp_path / "model.safetensors", header, data)
    with pytest.raises(SafetensorsError) as e:
        TensorIndex(str(tmp_path))
    assert needle in str(e.value)


def test_truncated_files(tmp_path):
    (tmp_path / "model.safetensors").write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too small"):
        TensorIndex(str(tmp_path))
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="header overruns"):
        TensorIndex(str(tmp_path))
    os.remove(tmp_path / "model.safetensors")
    with pytest.raises(SafetensorsError, match="no .safetensors files"):
        TensorIndex(str(tmp_path))


def test_several_files_are_merged(tmp_path):
    w = _state(TINY_A)
    names = sorted(w)
    os.makedirs(tmp_path / "m")
    write_state_dict(str(tmp_path / "m" / "model-00001-of-00002.safetensors"), {k: w[k] for k in names[:7]})
    write_state_dict(str(tmp_path / "m" / "model-00002-of-00002.safetensors"), {k: w[k] for k in names[7:]})
    with open(tmp_path / "m" / "config.json", "w") as f:
        json.dump(TINY_A, f)
    m = build_llama(parse_config(TINY_A))
    load_model_weights(m, str(tmp_path / "m"), CPU32)
    assert torch.equal(m.final_norm.weight, w["model.norm.weight"])
