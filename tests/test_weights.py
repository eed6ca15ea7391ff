"""Weights: safetensors by name, one error for everything wrong, the random-weights mode."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import plain_llama as P
from tiny import TINY_A, TINY_B, make_model
from xyntetik_runner_amd.config import config_from_dict
from xyntetik_runner_amd.engine.model import Model
from xyntetik_runner_amd.parts.base import ParamSpec
from xyntetik_runner_amd.weights import (SafetensorsError, SafetensorsStore, WeightError, check_against,
                                         load_tensors, save_safetensors, target_dtype, write_random_model)


def expected_for(raw):
    arch, cfg = config_from_dict(raw)
    return Model.expected_tensors(arch.build_spec(cfg))


def test_round_trip_and_foreign_reader(tmp_path):
    t = {"a.weight": torch.randn(3, 5).to(torch.bfloat16), "b": torch.arange(7, dtype=torch.int32),
         "c": torch.randn(4, dtype=torch.float32)}
    path = str(tmp_path / "x.safetensors")
    save_safetensors(path, t)
    st = SafetensorsStore([path])
    assert sorted(st.names()) == ["a.weight", "b", "c"]
    for k, v in t.items():
        assert torch.equal(st.tensor(k), v) and st.dtype(k) == v.dtype and st.shape(k) == tuple(v.shape)
    from safetensors.torch import load_file      # an independent reader agrees
    other = load_file(path)
    for k, v in t.items():
        assert torch.equal(other[k], v)
    st.close()


def test_random_model_is_reproducible_and_seeded(tmp_path):
    a1 = make_model("A", str(tmp_path / "a1"))
    a2 = make_model("A", str(tmp_path / "a2"))
    w1, w2 = P.load_folder(a1)[1], P.load_folder(a2)[1]
    assert sorted(w1) == sorted(w2) and all(np.array_equal(w1[k], w2[k]) for k in w1)
    write_random_model(TINY_A, str(tmp_path / "a3"), seed=5)
    w3 = P.load_folder(str(tmp_path / "a3"))[1]
    assert not np.array_equal(w1["model.layers.0.mlp.up_proj.weight"], w3["model.layers.0.mlp.up_proj.weight"])
    q = w1["model.layers.1.self_attn.q_proj.weight"]
    assert abs(q.std() - 0.02) < 0.003 and abs(q.mean()) < 0.003
    assert np.all(w1["model.norm.weight"] == 1.0)
    b = P.load_folder(make_model("B", str(tmp_path / "b")))[1]
    nb = b["model.layers.2.input_layernorm.weight"]
    assert 0.03 < nb.std() < 0.2 and "lm_head.weight" not in b          # tied: no head tensor
    st = SafetensorsStore.open_folder(str(tmp_path / "b"))
    assert st.dtype("model.norm.weight") == torch.float32               # stored in 32 bits
    assert st.dtype("model.embed_tokens.weight") == torch.bfloat16
    st.close()


def test_dtype_rule():
    m, v, i = ParamSpec((2, 2)), ParamSpec((2,), role="vector"), ParamSpec((2,), role="int")
    bf, f32 = torch.bfloat16, torch.float32
    assert target_dtype(m, f32, bf) == bf and target_dtype(m, bf, bf) == bf
    assert target_dtype(v, f32, bf) == f32          # a tensor stored in 32-bit stays so
    assert target_dtype(v, bf, bf) == bf
    assert target_dtype(i, torch.int64, bf) == torch.int32
    assert target_dtype(m, bf, f32) == f32 and target_dtype(v, bf, f32) == f32


def test_one_error_lists_missing_unexpected_and_wrong(tmp_path):
    d = make_model("A", str(tmp_path / "m"))
    st = SafetensorsStore.open_folder(d)
    state = {n: st.tensor(n).clone() for n in st.names()}
    st.close()
    del state["model.layers.1.mlp.down_proj.weight"]
    del state["model.norm.weight"]
    state["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)   # wrong rows
    state["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(64, 64, dtype=torch.int32)      # wrong dtype
    state["model.layers.7.extra.weight"] = torch.zeros(1)
    state["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)                        # ignored buffer
    save_safetensors(os.path.join(d, "model.safetensors"), state)
    st = SafetensorsStore.open_folder(d)
    with pytest.raises(WeightError) as e:
        load_tensors(st, expected_for(TINY_A), torch.float32, torch.device("cpu"))
    st.close()
    err = e.value
    assert err.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert len(err.wrong) == 2 and "[16, 64]" in err.wrong[0] + err.wrong[1] and "[32, 64]" in str(err)
    msg = str(err)
    for needle in ("missing", "unexpected", "wrong shape", "k_proj", "o_proj", "extra"):
        assert needle in msg


def test_tied_model_refuses_a_head_tensor_and_untied_needs_it():
    exp_b = expected_for(TINY_B)
    assert "lm_head.weight" not in exp_b
    names = list(exp_b) + ["lm_head.weight"]
    with pytest.raises(WeightError) as e:
        check_against(exp_b, names, lambda n: exp_b[n].shape if n in exp_b else (384, 96), lambda n: torch.bfloat16)
    assert e.value.unexpected == ["lm_head.weight"]
    exp_a = expected_for(TINY_A)
    names = [n for n in exp_a if n != "lm_head.weight"]
    with pytest.raises(WeightError) as e:
        check_against(exp_a, names, lambda n: exp_a[n].shape, lambda n: torch.bfloat16)
    assert e.value.missing == ["lm_head.weight"]


def test_container_refusals(tmp_path):
    p = str(tmp_path / "t.safetensors")
    save_safetensors(p, {"w": torch.ones(8, 8)})
    raw = open(p, "rb").read()
    # truncated data
    open(p, "wb").write(raw[:-16])
    with pytest.raises(SafetensorsError) as e:
        SafetensorsStore([p])
    assert "truncated" in str(e.value) or "ends at" in str(e.value)
    # header longer than the file
    open(p, "wb").write(struct.pack("<Q", 1 << 40) + raw[8:])
    with pytest.raises(SafetensorsError):
        SafetensorsStore([p])
    # size does not match shape
    hdr = json.dumps({"w": {"dtype": "F32", "shape": [8, 8], "data_offsets": [0, 100]}}).encode()
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 256)
    with pytest.raises(SafetensorsError) as e:
        SafetensorsStore([p])
    assert "256 bytes" in str(e.value)
    # a name twice
    hdr = b'{"w":{"dtype":"F32","shape":[1],"data_offsets":[0,4]},"w":{"dtype":"F32","shape":[1],"data_offsets":[4,8]}}'
    open(p, "wb").write(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(SafetensorsError) as e:
        SafetensorsStore([p])
    assert "twice" in str(e.value)
    with pytest.raises(SafetensorsError):
        SafetensorsStore.open_folder(str(tmp_path / "empty"))


def test_sharded_folder(tmp_path):
    d = tmp_path / "s"
    d.mkdir()
    save_safetensors(str(d / "p1.safetensors"), {"a": torch.ones(2)})
    save_safetensors(str(d / "p2.safetensors"), {"b": torch.zeros(3)})
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"a": "p1.safetensors", "b": "p2.safetensors"}}))
    st = SafetensorsStore.open_folder(str(d))
    assert sorted(st.names()) == ["a", "b"] and st.tensor("b").numel() == 3
    st.close()
