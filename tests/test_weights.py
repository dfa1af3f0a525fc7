"""Weights by name from safetensors: round trip with the safetensors package,
kept dtypes, and one error that lists every missing, unexpected and mis-shaped
tensor (the reference panics on the first missing one, src/arch/mod.rs:59-61)."""
import json
import os
import struct

import pytest
import torch

from llm_rs_amd import Engine, LlamaConfig, WeightError, load_tensors, random_model_tensors, write_model_folder
from llm_rs_amd.engine import Model
from llm_rs_amd.weights import SafetensorsError, SafetensorsFile, stored_dtype, write_safetensors
from tiny_configs import TINY_A, TINY_B


def test_round_trip_with_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn(5, 7, generator=g).bfloat16(), "b": torch.randn(3, generator=g),
               "ids": torch.arange(6, dtype=torch.int64).view(2, 3), "half": torch.randn(4, generator=g).half(),
               "empty": torch.zeros(0, 4)}
    ours, theirs = str(tmp_path / "ours.safetensors"), str(tmp_path / "theirs.safetensors")
    write_safetensors(ours, tensors)
    st.save_file(tensors, theirs)
    back = st.load_file(ours)
    f = SafetensorsFile(theirs)
    assert sorted(f.names()) == sorted(tensors)
    for name, t in tensors.items():
        assert torch.equal(back[name], t) and torch.equal(f.tensor(name), t) and f.tensor(name).dtype == t.dtype


def test_kept_dtypes():
    assert stored_dtype(torch.bfloat16) == torch.bfloat16 and stored_dtype(torch.float16) == torch.bfloat16
    assert stored_dtype(torch.float32) == torch.float32          # what is stored in 32-bit stays so
    assert stored_dtype(torch.int64) == torch.int32 and stored_dtype(torch.uint8) == torch.int32
    # a float16 file keeps its own values when the engine computes in 32-bit
    assert stored_dtype(torch.float16, torch.float32) == torch.float32
    assert stored_dtype(torch.bfloat16, torch.float32) == torch.bfloat16


def test_load_keeps_32_bit_and_makes_int32(tmp_path):
    write_safetensors(str(tmp_path / "model.safetensors"),
                      {"w": torch.ones(2, 2).bfloat16(), "n": torch.ones(2), "t": torch.arange(3)})
    got = load_tensors(str(tmp_path), {"w": (2, 2), "n": (2,), "t": (3,)}, log=False)
    assert got["w"].dtype == torch.bfloat16 and got["n"].dtype == torch.float32 and got["t"].dtype == torch.int32


def test_one_error_lists_everything(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_A)
    tensors = random_model_tensors(cfg, 0)
    del tensors["model.layers.0.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.1.self_attn.q_proj.weight"] = torch.zeros(64, 63).bfloat16()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)   # left unread, not an error
    tensors["model.layers.0.mlp.gate_proj.bias"] = torch.zeros(192)
    tensors["model.layers.9.input_layernorm.weight"] = torch.zeros(64)
    write_model_folder(str(tmp_path), cfg, tensors)
    with pytest.raises(WeightError) as e:
        Engine.from_folder(str(tmp_path), device="cpu", num_pages=4)
    err = e.value
    assert err.missing == ["model.layers.0.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.mlp.gate_proj.bias", "model.layers.9.input_layernorm.weight"]
    assert err.wrong_shape == [("model.layers.1.self_attn.q_proj.weight", (64, 64), (64, 63))]
    text = str(err)
    for piece in ("missing (2)", "unexpected (2)", "expected [64, 64] got [64, 63]", "model.norm.weight"):
        assert piece in text


def test_tensors_an_architecture_may_carry_unused_are_left_unread(tmp_path, capsys):
    """Older Llama files store the rotation's frequencies, files of tied models may repeat the token
    table as lm_head.weight: the folder loads, and a line says what was not read."""
    cfg = LlamaConfig.from_dict(TINY_A)                 # tied
    tensors = random_model_tensors(cfg, 0)
    for i in range(2):
        tensors[f"model.layers.{i}.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    write_model_folder(str(tmp_path / "a"), cfg, tensors)
    from emulated_kernels import EmulatedKernels
    from llm_rs_amd import use_kernels
    with use_kernels(EmulatedKernels()):
        eng = Engine.from_folder(str(tmp_path / "a"), device="cpu", dtype="float32", num_pages=8, page_size=4)
        assert eng.generate([[1, 2, 3]], max_new_tokens=2)
    said = capsys.readouterr().err
    assert "left unread" in said and "rotary_emb.inv_freq" in said and "lm_head.weight" in said
    # an untied model's files have no business holding a second head under another name
    cfg_b = LlamaConfig.from_dict(TINY_B)
    tensors = random_model_tensors(cfg_b, 0)
    tensors["output.weight"] = torch.zeros(2)
    with pytest.raises(WeightError, match="unexpected"):
        Model(cfg_b.model_spec(), torch.float32, "cpu").load(tensors)


def test_float16_file_is_exact_under_a_float32_engine(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_A)
    g = torch.Generator().manual_seed(0)
    tensors = {n: (t.float() + 1e-3 * torch.randn(t.shape, generator=g)).half() for n, t in random_model_tensors(cfg, 0).items()}
    write_model_folder(str(tmp_path), cfg, tensors)
    want = {n: tuple(t.shape) for n, t in tensors.items()}
    exact = load_tensors(str(tmp_path), want, log=False, compute=torch.float32)
    rounded = load_tensors(str(tmp_path), want, log=False, compute=torch.bfloat16)
    name = "model.layers.0.mlp.down_proj.weight"
    assert exact[name].dtype == torch.float32 and torch.equal(exact[name], tensors[name].float())
    assert rounded[name].dtype == torch.bfloat16 and not torch.equal(rounded[name].float(), tensors[name].float())
    from emulated_kernels import EmulatedKernels
    from llm_rs_amd import use_kernels
    with use_kernels(EmulatedKernels()):
        eng = Engine.from_folder(str(tmp_path), device="cpu", dtype="float32", num_pages=8, page_size=4)
    assert torch.equal(eng.model.blocks[0].feed_forward.w_down, tensors[name].float())


def test_untied_model_needs_its_head():
    cfg = LlamaConfig.from_dict(TINY_B)
    tensors = random_model_tensors(cfg, 0)
    del tensors["lm_head.weight"]
    with pytest.raises(WeightError, match="lm_head.weight"):
        Model(cfg.model_spec(), torch.float32, "cpu").load(tensors)


def test_broken_files(tmp_path):
    p = tmp_path / "model.safetensors"
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        load_tensors(str(tmp_path), {}, log=False)
    p.write_bytes(b"\x01")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    head = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(head)) + head + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="do not fit"):
        SafetensorsFile(str(p))
    head = json.dumps({"w": {"dtype": "Q4_K", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(head)) + head + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="unknown dtype"):
        SafetensorsFile(str(p))


def test_sharded_folder(tmp_path):
    a, b = torch.ones(2, 2).bfloat16(), torch.zeros(3)
    write_safetensors(str(tmp_path / "s1.safetensors"), {"a": a})
    write_safetensors(str(tmp_path / "s2.safetensors"), {"b": b})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    got = load_tensors(str(tmp_path), {"a": (2, 2), "b": (3,)}, log=False)
    assert torch.equal(got["a"], a) and torch.equal(got["b"], b)


def test_random_weights_are_a_function_of_seed_and_name(tmp_path):
    cfg = LlamaConfig.from_dict(TINY_B)
    t0, t0b, t1 = random_model_tensors(cfg, 0), random_model_tensors(cfg, 0), random_model_tensors(cfg, 1)
    for name in t0:
        assert torch.equal(t0[name], t0b[name])
        assert not torch.equal(t0[name], t1[name])
    norm = t0["model.layers.0.input_layernorm.weight"].float()
    w = t0["model.layers.0.mlp.gate_proj.weight"].float()
    assert abs(float(norm.mean()) - 1.0) < 0.05 and 0.05 < float(norm.std()) < 0.15
    assert abs(float(w.mean())) < 2e-3 and 0.018 < float(w.std()) < 0.022
    write_model_folder(str(tmp_path / "m"), cfg, t0)
    assert sorted(os.listdir(tmp_path / "m")) == ["config.json", "model.safetensors"]
    assert LlamaConfig.from_dict(json.load(open(tmp_path / "m" / "config.json"))) == cfg
