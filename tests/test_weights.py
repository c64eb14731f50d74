"""Safetensors reading and writing, random-weights mode, and the one error that lists what is
wrong with a checkpoint (no GPU)."""
import json
import os

import numpy as np
import pytest
import torch

from burn_lm_amd import registry
from burn_lm_amd.engine.model import Model
from burn_lm_amd.weights import loader, safetensors_io as st
from helpers import TINY_A, TINY_B, make_folder


def _specs(cfg):
    a = registry.architecture_of(cfg)
    return a, Model(a.plan(a.read_config(cfg), None)).tensor_specs()


def test_written_folder_is_read_by_the_library_reader_and_ours(tmp_path):
    from safetensors.torch import load_file
    d = make_folder(tmp_path, TINY_B, seed=1)
    lib = load_file(os.path.join(d, "model.safetensors"))
    ours = st.open_folder(d)
    assert set(lib) == set(ours)
    for n, t in lib.items():
        assert t.dtype == torch.bfloat16
        assert torch.equal(ours[n].tensor(n), t)
    assert json.load(open(os.path.join(d, "config.json")))["hidden_size"] == 144


def test_file_written_by_the_library_is_read_by_ours(tmp_path):
    from safetensors.torch import save_file
    t = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.ones(4, dtype=torch.bfloat16),
         "c": torch.arange(5, dtype=torch.int64)}
    save_file(t, str(tmp_path / "model.safetensors"))
    f = st.open_folder(str(tmp_path))
    for n in t:
        assert torch.equal(f[n].tensor(n), t[n]) and f[n].dtype(n) == t[n].dtype


def test_random_mode_is_seeded(tmp_path):
    a = st.open_folder(make_folder(tmp_path / "a", TINY_A, seed=3))
    b = st.open_folder(make_folder(tmp_path / "b", TINY_A, seed=3))
    c = st.open_folder(make_folder(tmp_path / "c", TINY_A, seed=4))
    n = "model.layers.1.mlp.up_proj.weight"
    assert torch.equal(a[n].tensor(n), b[n].tensor(n))
    assert not torch.equal(a[n].tensor(n), c[n].tensor(n))
    w = a[n].tensor(n).float()
    assert abs(float(w.std()) - 0.08) < 0.01 and w.shape == (176, 64)
    assert "lm_head.weight" not in a  # tied


def test_loads_every_tensor_the_model_asks_for(tmp_path):
    d = make_folder(tmp_path, TINY_B, seed=1)
    _, specs = _specs(TINY_B)
    t = loader.load(d, specs, torch.bfloat16, "cpu")
    assert set(t) == set(specs)
    assert all(v.dtype == torch.bfloat16 for v in t.values())
    t32 = loader.load(d, specs, torch.float32, "cpu")
    assert all(v.dtype == torch.float32 for v in t32.values())
    n = "model.layers.2.self_attn.k_proj.weight"
    assert t[n].shape == (24, 144) and torch.equal(t32[n], t[n].float())


def test_a_tensor_stored_in_32_bits_stays_so(tmp_path):
    d = make_folder(tmp_path, TINY_A, seed=0)
    f = st.open_folder(d)
    tensors = [(n, f[n].tensor(n).clone()) for n in f]
    tensors = [(n, t.float() if n.endswith("norm.weight") else t) for n, t in tensors]
    tensors.append(("model.layers.0.self_attn.rotary_emb.inv_freq", torch.ones(8)))
    st.write_file(os.path.join(d, "model.safetensors"), tensors)
    _, specs = _specs(TINY_A)
    a = registry.architecture("llama")
    plan = a.plan(a.read_config(TINY_A), None)
    t = loader.load(d, specs, torch.bfloat16, "cpu", plan.ignorable_tensors)
    assert t["model.norm.weight"].dtype == torch.float32
    assert t["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = make_folder(tmp_path, TINY_B, seed=1)
    f = st.open_folder(d)
    tensors = {n: f[n].tensor(n).clone() for n in f}
    del tensors["model.layers.1.mlp.down_proj.weight"]
    del tensors["lm_head.weight"]
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(144, dtype=torch.bfloat16)
    tensors["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(48, 144, dtype=torch.bfloat16)
    tensors["model.norm.weight"] = torch.zeros(144, dtype=torch.int32)
    st.write_file(os.path.join(d, "model.safetensors"), tensors.items())
    _, specs = _specs(TINY_B)
    with pytest.raises(loader.WeightError) as e:
        loader.load(d, specs, torch.bfloat16, "cpu")
    err = e.value
    assert err.missing == ["lm_head.weight", "model.layers.1.mlp.down_proj.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert err.wrong_shape == [("model.layers.2.self_attn.k_proj.weight", (48, 144), (24, 144))]
    assert err.wrong_kind and err.wrong_kind[0][0] == "model.norm.weight"
    msg = str(err)
    for word in ("missing tensors (2)", "lm_head.weight", "unexpected tensors (1)", "q_proj.bias",
                 "[48, 144]", "[24, 144]", "model.norm.weight"):
        assert word in msg


def test_broken_files_are_refused(tmp_path):
    with pytest.raises(st.SafetensorsError, match="neither"):
        st.open_folder(str(tmp_path))
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"\x00\x01")
    with pytest.raises(st.SafetensorsError, match="too short"):
        st.open_folder(str(tmp_path))
    p.write_bytes((1 << 40).to_bytes(8, "little") + b"{}")
    with pytest.raises(st.SafetensorsError, match="header length"):
        st.open_folder(str(tmp_path))
    h = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(len(h).to_bytes(8, "little") + h + b"\0" * 8)
    with pytest.raises(st.SafetensorsError, match="offsets"):
        st.open_folder(str(tmp_path))


def test_sharded_folder(tmp_path):
    st.write_file(str(tmp_path / "s1.safetensors"), [("a", torch.ones(2))])
    st.write_file(str(tmp_path / "s2.safetensors"), [("b", torch.zeros(3))])
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    f = st.open_folder(str(tmp_path))
    assert f["a"].tensor("a").tolist() == [1, 1] and f["b"].shape("b") == (3,)


def test_random_weights_are_a_function_of_seed_name_and_index():
    """Every value depends on (seed, tensor name, element index) alone: the same tensor comes out
    whole or in pieces, first or last, and another seed or name gives another one; the values are
    normal to within what an initialisation can tell."""
    from burn_lm_amd.weights import random_init as R
    key = R.tensor_key(3, "a.weight")
    whole = R.standard_normal(key, 0, 5000)
    assert torch.equal(whole[1234:1300], R.standard_normal(key, 1234, 66))
    assert not torch.equal(whole[:100], R.standard_normal(R.tensor_key(4, "a.weight"), 0, 100))
    assert not torch.equal(whole[:100], R.standard_normal(R.tensor_key(3, "b.weight"), 0, 100))
    z = R.standard_normal(key, 0, 400000).double()
    assert abs(float(z.mean())) < 0.01 and abs(float(z.std()) - 1) < 0.01
    assert abs(float((z ** 4).mean()) - 3) < 0.2 and float(z.abs().max()) > 3.5
    a = R.make_tensor("w", (70, 33), "matrix", seed=9, std=0.02)
    b = R.make_tensor("w", (70, 33), "matrix", seed=9, std=0.02)
    assert a.dtype == torch.bfloat16 and torch.equal(a, b) and 0.018 < float(a.float().std()) < 0.022
    assert torch.equal(R.make_tensor("n", (8,), "norm", seed=9), torch.ones(8, dtype=torch.bfloat16))
    table = R.make_tensor("t", (1000,), R.IntegerTable(7), seed=9)
    assert table.dtype == torch.int32 and set(table.tolist()) == set(range(7))
    with pytest.raises(ValueError, match="role"):
        R.make_tensor("x", (3,), "matrices", seed=0)


def test_the_range_initialiser_is_the_references_fixture(tmp_path):
    """crates/burn-lm-llama/src/lib.rs:142-148: arange(n) * (max - min) / n + min, over a linear weight
    in the reference's [d_in, d_out] order.  As a Meta-named checkpoint of the reference's tiny test
    model it holds exactly the tensors the reference's whole-model vector is computed from
    (crates/burn-lm-llama/src/nn/transformer.rs:299-349)."""
    import burn_lm_amd
    from burn_lm_amd.weights.random_init import Range
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=8, intermediate_size=16, num_hidden_layers=2,
               num_attention_heads=2, num_key_value_heads=1, vocab_size=8, rms_norm_eps=1e-5, rope_theta=10000.0,
               tie_word_embeddings=False, max_position_embeddings=64)
    folder = burn_lm_amd.write_random_model(str(tmp_path), cfg, init=Range(0.0, 5.0), names="meta", dtype=torch.float32)
    f = st.open_folder(folder)
    r = lambda *s: torch.arange(int(np.prod(s)), dtype=torch.float64).mul(5.0 / int(np.prod(s))).reshape(*s)
    assert torch.equal(f["tok_embeddings.weight"].tensor("tok_embeddings.weight"), r(8, 8).float())
    assert torch.equal(f["norm.weight"].tensor("norm.weight"), r(8).float())
    wk = f["layers.1.attention.wk.weight"].tensor("layers.1.attention.wk.weight")
    assert wk.shape == (4, 8) and torch.equal(wk, r(8, 4).T.contiguous().float())      # [d_out, d_in] of a [d_in, d_out] ramp
    w2 = f["layers.0.feed_forward.w2.weight"].tensor("layers.0.feed_forward.w2.weight")
    assert w2.shape == (8, 16) and torch.equal(w2, r(16, 8).T.contiguous().float())
    assert "output.weight" in f and "layers.1.ffn_norm.weight" in f and len(f) == 3 + 2 * 9
