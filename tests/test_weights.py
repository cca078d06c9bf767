"""Safetensors by name, the whole-checkpoint check, stored precision, random weights."""
import json
import os

import pytest
import torch

import inferllm_amd as I
from inferllm_amd.engine import DecoderModel, expected_tensors
from inferllm_amd.weights import (SafetensorsError, SafetensorsFile, WeightsError, check_names,
                                  kept_dtype, load_named_tensors, open_model_files,
                                  random_tensor, write_safetensors, TensorWant)
from tiny import TINY_A, TINY_B, TINY_C, make_model_dir, read_weights


def test_file_round_trip_all_dtypes(tmp_path):
    g = torch.Generator().manual_seed(0)
    tensors = {"a.f32": torch.randn(3, 5, generator=g), "b.bf16": torch.randn(7, generator=g).bfloat16(),
               "c.f16": torch.randn(2, 2, 2, generator=g).half(), "d.i64": torch.arange(6).reshape(2, 3),
               "e.i32": torch.arange(4, dtype=torch.int32), "f.empty": torch.zeros(0, 4)}
    p = str(tmp_path / "t.safetensors")
    write_safetensors(p, tensors.items(), {"k": "v"})
    f = SafetensorsFile(p)
    assert f.metadata == {"k": "v"} and set(f.names()) == set(tensors)
    for n, t in tensors.items():
        got = f.read(n)
        assert got.dtype == t.dtype and got.shape == t.shape and torch.equal(got, t)
    f.close()


def test_file_is_readable_by_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    t = {"x": torch.randn(4, 3).bfloat16(), "y": torch.arange(5, dtype=torch.int32)}
    p = str(tmp_path / "t.safetensors")
    write_safetensors(p, t.items())
    back = st.load_file(p)
    assert all(torch.equal(back[k], v) for k, v in t.items())
    st.save_file(t, str(tmp_path / "u.safetensors"))
    f = SafetensorsFile(str(tmp_path / "u.safetensors"))
    assert all(torch.equal(f.read(k), v) for k, v in t.items())


def test_broken_files(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(p))
    p.write_bytes((10**9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(str(p))
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(len(hdr).to_bytes(8, "little") + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 16 bytes"):
        SafetensorsFile(str(p))
    with pytest.raises(SafetensorsError, match="no model.safetensors"):
        open_model_files(str(tmp_path / "nowhere"))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = I.config_from_dict(TINY_A)
    d = make_model_dir(tmp_path, TINY_A, seed=1)
    w = read_weights(d)
    del w["model.layers.1.mlp.up_proj.weight"], w["model.norm.weight"]
    w["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 32)
    w["lm_head.weight"] = torch.zeros(255, 64)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)     # ignored by suffix
    w["something.else"] = torch.zeros(2)
    w["model.embed_tokens.weight"] = torch.zeros(256, 64, dtype=torch.int32)
    write_safetensors(os.path.join(d, "model.safetensors"), w.items())
    model = DecoderModel(cfg.to_spec())
    with pytest.raises(WeightsError) as e:
        load_named_tensors(d, model.wants(), torch.float32, "cpu", cfg.to_spec().ignored_tensor_suffixes)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["something.else"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["lm_head.weight", "model.layers.0.self_attn.q_proj.weight"]
    assert [n for n, _ in err.wrong_dtype] == ["model.embed_tokens.weight"]
    msg = str(err)
    for s in ("missing tensors (2)", "unexpected tensors (1)", "something.else",
              "lm_head.weight is [255, 64], the model needs [256, 64]"):
        assert s in msg


def test_precision_in_memory():
    """Matrices take the engine's dtype as the reference gives every tensor the runtime type of
    its file code (src/core/graph.cpp:216-231); tensors marked keep_stored keep the file's."""
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert kept_dtype(bf, "float", bf) == bf
    assert kept_dtype(f32, "float", bf) == bf           # a matrix is rounded to the engine's dtype
    assert kept_dtype(f16, "float", bf) == bf
    assert kept_dtype(f32, "float", bf, keep_stored=True) == f32   # stored in 32-bit stays so
    assert kept_dtype(f16, "float", bf, keep_stored=True) == f32   # widened exactly
    assert kept_dtype(bf, "float", bf, keep_stored=True) == bf
    assert kept_dtype(bf, "float", f32) == f32          # a float32 engine widens everything
    assert kept_dtype(f16, "float", f32, keep_stored=True) == f32
    assert kept_dtype(torch.int64, "int", bf) == torch.int32


def test_mixed_precision_folder(tmp_path):
    cfg = I.config_from_dict(TINY_A)
    d = make_model_dir(tmp_path, TINY_A, seed=2, dtype=torch.bfloat16)
    w = read_weights(d)
    w["model.norm.weight"] = w["model.norm.weight"].float()
    write_safetensors(os.path.join(d, "model.safetensors"), w.items())
    model = DecoderModel(cfg.to_spec())
    t = load_named_tensors(d, model.wants(), torch.bfloat16, "cpu")
    assert t["model.norm.weight"].dtype == torch.float32     # a norm weight keeps its 32 bits
    assert t["model.layers.0.input_layernorm.weight"].dtype == torch.bfloat16
    assert t["lm_head.weight"].dtype == torch.bfloat16
    t32 = load_named_tensors(d, model.wants(), torch.float32, "cpu")
    assert all(v.dtype == torch.float32 for v in t32.values())
    assert torch.equal(t32["lm_head.weight"], t["lm_head.weight"].float())


@pytest.mark.parametrize("stored", [torch.float16, torch.float32])
def test_float16_and_float32_folders_in_a_bfloat16_engine(tmp_path, stored):
    """Every matrix is rounded to bfloat16 to nearest even; norm weights stay 32-bit; with
    keep_stored nothing is rounded."""
    cfg = I.config_from_dict(TINY_A)
    d = make_model_dir(tmp_path, TINY_A, seed=5, dtype=stored)
    w = read_weights(d)
    model = DecoderModel(cfg.to_spec())
    t = load_named_tensors(d, model.wants(), torch.bfloat16, "cpu")
    for n, v in t.items():
        if v.dim() == 2:
            assert v.dtype == torch.bfloat16, n
            assert torch.equal(v, w[n].float().to(torch.bfloat16)), n
        else:
            assert v.dtype == torch.float32 and torch.equal(v, w[n].float()), n
    # ties go to the even neighbour: 1 + 2^-8 lies midway between 1 and 1 + 2^-7
    x = torch.tensor([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8], dtype=torch.float32)
    assert x.to(torch.bfloat16).float().tolist() == [1.0, 1.0 + 2.0 ** -6]
    kept = load_named_tensors(d, model.wants(), torch.bfloat16, "cpu", keep_stored=True)
    assert all(v.dtype == torch.float32 and torch.equal(v, w[n].float()) for n, v in kept.items())


def test_sharded_folder(tmp_path):
    cfg = I.config_from_dict(TINY_A)
    d = make_model_dir(tmp_path, TINY_A, seed=3)
    w = read_weights(d)
    names = sorted(w)
    half = len(names) // 2
    os.remove(os.path.join(d, "model.safetensors"))
    write_safetensors(os.path.join(d, "m-1.safetensors"), [(n, w[n]) for n in names[:half]])
    write_safetensors(os.path.join(d, "m-2.safetensors"), [(n, w[n]) for n in names[half:]])
    wm = {n: ("m-1.safetensors" if i < half else "m-2.safetensors") for i, n in enumerate(names)}
    with open(os.path.join(d, "model.safetensors.index.json"), "w") as f:
        json.dump({"weight_map": wm}, f)
    t = load_named_tensors(d, DecoderModel(cfg.to_spec()).wants(), torch.float32, "cpu")
    assert set(t) == set(w) and all(torch.equal(t[n], w[n]) for n in w)


def test_tied_head_needs_no_tensor_of_its_own(tmp_path):
    cfg = I.config_from_dict(TINY_C)
    wants = expected_tensors(cfg.to_spec())
    assert wants["lm_head.weight"].optional and not wants["model.embed_tokens.weight"].optional
    d = make_model_dir(tmp_path, TINY_C, seed=4)
    assert "lm_head.weight" not in read_weights(d)
    model = DecoderModel(cfg.to_spec())
    model.load(load_named_tensors(d, model.wants(), torch.float32, "cpu"))
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()


def test_random_weights_follow_the_rule_and_the_seed(tmp_path):
    a = make_model_dir(tmp_path / "a", TINY_B, seed=5)
    b = make_model_dir(tmp_path / "b", TINY_B, seed=5)
    c = make_model_dir(tmp_path / "c", TINY_B, seed=6)
    wa, wb, wc = read_weights(a), read_weights(b), read_weights(c)
    assert all(torch.equal(wa[n], wb[n]) for n in wa)
    assert not torch.equal(wa["lm_head.weight"], wc["lm_head.weight"])
    lin = wa["model.layers.0.mlp.gate_proj.weight"]
    assert abs(float(lin.std()) - 0.02) < 0.002 and abs(float(lin.mean())) < 0.002
    nw = wa["model.layers.2.input_layernorm.weight"]
    assert abs(float(nw.mean()) - 1.0) < 0.01 and 0.002 < float(nw.std()) < 0.03
    # a tensor's values depend on (seed, name) only, not on the model around it
    want = TensorWant((320, 96))
    assert torch.equal(random_tensor(5, "lm_head.weight", want, torch.float32), wa["lm_head.weight"])
    cfg = json.load(open(os.path.join(a, "config.json")))
    assert cfg["architectures"] == ["LlamaForCausalLM"] and cfg["torch_dtype"] == "float32"
    bf = make_model_dir(tmp_path / "d", TINY_B, seed=5, dtype=torch.bfloat16)
    assert torch.equal(read_weights(bf)["lm_head.weight"], wa["lm_head.weight"].bfloat16())
