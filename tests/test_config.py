"""Configuration and registry (no GPU)."""
import json

import pytest

import burn_lm_amd  # noqa: F401
from burn_lm_amd import registry
from burn_lm_amd.config.llama import ConfigError, LlamaConfig, RopeScaling
from burn_lm_amd.config.presets import preset, presets
from helpers import TINY_A, TINY_B


def test_reads_every_size_from_its_keys():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (144, 384, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim) == (6, 1, 24)
    assert (c.vocab_size, c.max_position_embeddings) == (384, 384)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.tie_word_embeddings is False
    assert c.rope_scaling == RopeScaling(8.0, 1.0, 4.0, 32)


def test_defaults_are_the_references():
    # crates/burn-lm-llama/src/nn/llama/base.rs:54-62,254; nn/attention/mha.rs:191; nn/pos_encoding.rs:91-101
    d = {k: v for k, v in TINY_A.items() if k not in ("num_key_value_heads", "rms_norm_eps", "rope_theta",
                                                      "tie_word_embeddings")}
    c = LlamaConfig.from_dict(d)
    assert c.num_key_value_heads == c.num_attention_heads == 4
    assert c.head_dim == 16 and c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0
    assert c.tie_word_embeddings is False and c.rope_scaling is None
    c = LlamaConfig.from_dict({**TINY_A, "rope_scaling": {"rope_type": "llama3"}})
    assert c.rope_scaling == RopeScaling(8.0, 1.0, 4.0, 8192)
    # the older key name, and the spelled-out absence of scaling
    assert LlamaConfig.from_dict({**TINY_A, "rope_scaling": {"type": "llama3", "factor": 2}}).rope_scaling.factor == 2.0
    assert LlamaConfig.from_dict({**TINY_A, "rope_scaling": {"rope_type": "default"}}).rope_scaling is None


@pytest.mark.parametrize("key", ["hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                                 "vocab_size", "max_position_embeddings"])
def test_missing_size_names_the_key(key):
    d = dict(TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


@pytest.mark.parametrize("patch,word", [
    ({"num_key_value_heads": 3}, "num_key_value_heads"),
    ({"head_dim": 15}, "head_dim"),
    ({"hidden_size": "64"}, "hidden_size"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"attention_bias": True}, "attention_bias"),
    ({"mlp_bias": True}, "mlp_bias"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"eos_token_id": 999}, "999"),
    ({"rms_norm_eps": 0}, "rms_norm_eps"),
    ({"hidden_size": 66, "head_dim": None}, "head_dim"),
])
def test_bad_values_are_refused_with_their_key(patch, word):
    with pytest.raises(ConfigError, match=word):
        LlamaConfig.from_dict({**TINY_A, **patch})


def test_eos_may_be_one_id_or_a_list_and_round_trips():
    c = LlamaConfig.from_dict({**TINY_A, "eos_token_id": [1, 2]})
    assert c.eos_token_ids == (1, 2)
    assert LlamaConfig.from_dict({**TINY_A, "eos_token_id": 7}).eos_token_ids == (7,)
    assert LlamaConfig.from_dict(c.to_dict()) == c
    assert LlamaConfig.from_dict(LlamaConfig.from_dict(TINY_B).to_dict()) == LlamaConfig.from_dict(TINY_B)


def test_folder_errors(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        LlamaConfig.from_folder(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        LlamaConfig.from_folder(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    assert LlamaConfig.from_folder(str(tmp_path)).hidden_size == 64


def test_registry_maps_names_to_the_architecture():
    a = registry.architecture_of(TINY_A)
    assert a is registry.architecture("llama") is registry.architecture("LlamaForCausalLM")
    with pytest.raises(registry.RegistryError, match="LlamaForCausalLM"):
        registry.architecture("MambaForCausalLM")
    with pytest.raises(registry.RegistryError, match="names no architecture"):
        registry.architecture_of({"hidden_size": 1})
    assert registry.architecture_of({"architectures": ["Nope"], "model_type": "llama"}) is a
    with pytest.raises(registry.RegistryError, match="attention"):
        registry.part("mixer", "nope")


def test_plan_follows_the_configuration():
    a = registry.architecture("llama")
    cfg = a.read_config(TINY_B)
    plan = a.plan(cfg, None)
    assert len(plan.layers) == 3 and [p.layer for p in plan.order] == [0, 1, 2]
    m = plan.layers[1].mixer
    assert m.kind == "attention" and m.params["heads"] == 6 and m.params["kv_heads"] == 1 and m.params["head_dim"] == 24
    assert abs(m.params["scale"] - 24 ** -0.5) < 1e-15
    assert plan.layers[0].mixer_norm.params["eps"] == 1e-6
    assert plan.positions["rope"].params["pairing"] == "half"
    assert plan.head.names["weight"] == "lm_head.weight"
    tied = a.plan(a.read_config(TINY_A), None)
    assert tied.head.names["weight"] == tied.embedding.names["weight"]
    meta = a.plan(cfg, {"tok_embeddings.weight"})
    assert meta.positions["rope"].params["pairing"] == "interleaved"
    assert meta.layers[0].feed_forward.names["gate"] == "layers.0.feed_forward.w1.weight"


def test_presets_are_valid_configurations():
    for name in presets():
        c = LlamaConfig.from_dict(preset(name))
        assert c.num_hidden_layers > 0
    c = LlamaConfig.from_dict(preset("llama3.2-1b"))
    # crates/burn-lm-llama/src/nn/llama/base.rs:103-113
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads,
            c.intermediate_size, c.vocab_size) == (2048, 16, 32, 8, 8192, 128256)
    assert c.rope_scaling.factor == 32.0 and c.rope_theta == 500000.0
    # the two tiny shapes of the tests can be named from the command line as well: same sizes and options
    from helpers import TINY_A, TINY_B
    for name, tiny in (("tiny-a", TINY_A), ("tiny-b", TINY_B)):
        p = preset(name)
        for key, value in tiny.items():
            if key != "max_position_embeddings":      # the tests give themselves a longer context
                assert p[key] == value, (name, key)
    assert preset("tiny-a")["max_position_embeddings"] == 128 and preset("tiny-b")["max_position_embeddings"] == 96
    assert LlamaConfig.from_dict(preset("tiny-b")).head_dim == 24


def test_tokenizers_for_the_command_line(tmp_path):
    """Bytes by default; a tokenizer.json in the model folder is used when there is one, with the
    stop ids of the special tokens it defines (tiktoken.rs:12-15, 126-132)."""
    from burn_lm_amd.text.tokenizer import ByteTokenizer, FileTokenizer, for_folder
    t = for_folder(str(tmp_path), 256)
    assert isinstance(t, ByteTokenizer) and t.decode(t.encode("héllo")) == "héllo" and t.stop_ids() == [2]
    assert t.encode("a", bos=True, eos=True) == [0, 97, 1]
    with pytest.raises(ValueError, match="at least 256"):
        for_folder(str(tmp_path), 100)
    from tokenizers import Tokenizer, models, pre_tokenizers
    vocab = {"hello": 0, "world": 1, "[UNK]": 2, "<|begin_of_text|>": 3, "<|end_of_text|>": 4, "<|eot_id|>": 5}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="[UNK]"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.add_special_tokens(["<|begin_of_text|>", "<|end_of_text|>", "<|eot_id|>"])
    tok.save(str(tmp_path / "tokenizer.json"))
    from burn_lm_amd import registry
    special = registry.architecture("LlamaForCausalLM").special_tokens     # the architecture names them, not the tokenizer
    f = for_folder(str(tmp_path), 6, special)
    assert isinstance(f, FileTokenizer)
    assert f.encode("hello world") == [0, 1] and f.encode("hello", bos=True, eos=True) == [3, 0, 4]
    assert f.stop_ids() == [4, 5]            # <|eom_id|> is not in this file
    assert f.decode([3, 0, 1, 5]) == "hello world"
    bare = for_folder(str(tmp_path), 6)      # an architecture that names no special tokens: none begin, end or stop
    assert bare.stop_ids() == [] and bare.encode("hello", bos=True, eos=True) == [0]


def test_decode_attention_split_rule():
    """How many pieces a sequence's pages are cut into for the decode attention: never more pieces
    than pages, pieces of at least eight pages (two while the chip would be mostly idle), no more
    blocks than the target."""
    from burn_lm_amd.parts.attention import decode_splits
    # the targets follow the chip: on half as many compute units, half as many pieces
    assert decode_splits(64, 8, 64, compute_units=128) == 8 and decode_splits(64, 64, 64, compute_units=64) == 1
    # context 4096 (64 pages), 8 key-value heads: batch 1, 2, 4, 8, 16, 64
    assert [decode_splits(64, b * 8, 64) for b in (1, 2, 4, 8, 16, 32, 64)] == [16, 8, 8, 4, 2, 1, 1]
    # all blocks in one round, at most one per compute unit, also where the batch is no power of two
    assert [decode_splits(64, b * 8, 64) for b in (3, 5, 6, 7, 10, 12, 14, 20, 24)] == [8, 6, 5, 4, 3, 2, 2, 1, 1]
    assert [decode_splits(256, b * 8, 128) for b in (3, 5, 6, 10, 20)] == [10, 6, 5, 3, 1]
    for b in range(1, 40):
        for pages in (20, 64, 256, 2048):
            assert b * 8 * decode_splits(pages, b * 8, 64) <= 256 or decode_splits(pages, b * 8, 64) == 1
    assert decode_splits(256, 32 * 8, 64) == 1                                      # every compute unit has a block: no cutting
    assert decode_splits(64, 8, 128) == 16 and decode_splits(64, 64, 128) == 4      # wide heads: half the blocks
    assert decode_splits(1, 8, 64) == 1 and decode_splits(3, 8, 64) == 1 and decode_splits(8, 8, 64) == 1
    # short ranges stay whole: up to two pages per wavefront, three with heads up to 64
    assert decode_splits(12, 8, 64) == 1 and decode_splits(13, 8, 64) == 6 and decode_splits(8, 8, 128) == 1 and decode_splits(12, 8, 128) == 6
    # 11 and 16 pages of wide heads at batch 1, 2, 4, 8, 16: two pages a piece while blocks are few, whole from 64 blocks on
    assert [decode_splits(11, b * 8, 128) for b in (1, 2, 4, 8, 16)] == [5, 5, 4, 1, 1]
    assert [decode_splits(16, b * 8, 128) for b in (1, 2, 4, 8, 16)] == [8, 8, 4, 1, 1]
    assert [decode_splits(16, b * 8, 64) for b in (1, 2, 4, 8, 16)] == [8, 8, 4, 1, 1]
    assert decode_splits(17, 64, 64) == 2                                           # beyond 16 pages the range is cut again
    assert decode_splits(2048, 8, 64) == 32 and decode_splits(512, 8, 64) == 32     # a long context at batch 1: the cap
    for pages in (1, 2, 5, 8, 9, 31, 64, 100, 1000):
        for blocks in (1, 3, 8, 64, 500, 5000):
            for hd in (64, 128):
                n = decode_splits(pages, blocks, hd)
                assert 1 <= n <= pages
                assert n == 1 or pages // n >= 2


def test_command_line_random_models_delete(tmp_path, monkeypatch, capsys):
    """`random` writes a model folder into the models directory, `models` lists it, `delete` removes
    it and nothing outside the models directory."""
    import pytest
    from burn_lm_amd.cli.main import main
    monkeypatch.setenv("BURN_LM_AMD_MODELS", str(tmp_path / "models"))
    outside = tmp_path / "elsewhere"
    outside.mkdir()
    (outside / "config.json").write_text("{}")
    main(["random", "llama3.2-1b-test", "--name", "mine"])
    assert (tmp_path / "models" / "mine" / "model.safetensors").exists()
    capsys.readouterr()
    main(["models"])
    listing = capsys.readouterr().out
    assert "| mine" in listing and "run mine" in listing and "random llama3.2-1b-test" in listing
    with pytest.raises(SystemExit, match="not in the models directory"):
        main(["delete", "../elsewhere"])
    with pytest.raises(SystemExit, match="not in the models directory"):
        main(["delete", "absent"])
    main(["delete", "mine"])
    assert not (tmp_path / "models" / "mine").exists() and (outside / "config.json").exists()
    main(["random", "llama3.2-1b-test"])
    main(["random", "llama3.2-1b-test", "--name", "second", "--seed", "3"])
    main(["delete", "all"])
    assert sorted(p.name for p in (tmp_path / "models").iterdir()) == []


def test_text_comes_out_piece_by_piece_as_the_whole_would():
    """The streaming decoder against two tokenizers whose tokens cannot be decoded one by one: bytes
    (a character of several bytes spans tokens) and a word tokenizer that puts a space between the
    words of one call and none in front of the first (crates/burn-lm-llama/src/generation/streaming.rs:10-57)."""
    from burn_lm_amd.text.tokenizer import ByteTokenizer, StreamingDecoder

    text = "héllo wörld — ça va? 日本語"
    ids = ByteTokenizer().encode(text)
    dec = StreamingDecoder(ByteTokenizer())
    pieces = [dec.push(t) for t in ids]
    assert "".join(pieces) + dec.flush() == text
    assert all("�" not in p for p in pieces) and any(p == "" for p in pieces)   # half characters are held back

    class Words:
        vocab = ["the", "quick", "brown", "fox", ",", "jumps"]

        def decode(self, tokens):
            out = ""
            for i, t in enumerate(tokens):
                w = self.vocab[t]
                out += w if i == 0 or w == "," else " " + w
            return out

    ids = [0, 1, 2, 3, 4, 5, 0, 3]
    dec = StreamingDecoder(Words())
    pieces = [dec.push(t) for t in ids]
    assert "".join(pieces) + dec.flush() == Words().decode(ids) == "the quick brown fox, jumps the fox"
    assert pieces[1] == " quick"          # decoded alone it would have lost its space
    # tokens that end in the middle of a character at the end of the text come out with the flush
    dec = StreamingDecoder(ByteTokenizer())
    cut = ByteTokenizer().encode("aé")[:-1]
    assert [dec.push(t) for t in cut] == ["a", ""] and dec.flush() == "�"


def test_how_a_product_of_17_to_64_rows_is_cut():
    """Groups of about 2048 of K, 32 columns per block where that is one round of blocks on 256 compute
    units, a short K cut further until most units have a block; a tiny product is not cut at all (it
    then stays with the packed kernel)."""
    from burn_lm_amd.engine.runtime import rows_plan
    shapes = {"1b o": (2048, 2048), "1b down": (2048, 8192), "3b o": (3072, 3072), "3b down": (3072, 8192),
              "8b o": (4096, 4096), "8b down": (4096, 14336), "tiny": (72, 136), "narrow": (64, 1200)}
    got = {k: rows_plan(n, kk, 256) for k, (n, kk) in shapes.items()}
    assert got == {"1b o": (4, 32), "1b down": (4, 32), "3b o": (2, 32), "3b down": (4, 64), "8b o": (2, 32),
                   "8b down": (4, 64), "tiny": (1, 32), "narrow": (2, 32)}
    for n, kk in shapes.values():
        groups, columns = rows_plan(n, kk, 256)
        assert groups == 1 or kk // groups >= 512
        assert columns in (32, 64)
