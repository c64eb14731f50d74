"""The engine on the GPU against the plain implementation: long decoding, the first tokens of a
sequence, greedy generation through the entry point, faults that random weights would hide."""
import json
import os

import numpy as np
import pytest
import torch

import plain_llama as P
from helpers import TINIES, TINY_A, TOL, make_folder, random_tokens, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {k: make_folder(tmp_path_factory.mktemp("m" + k), cfg, seed) for k, (cfg, seed) in TINIES.items()}


def load(folder, dtype, **kw):
    from burn_lm_amd.engine.loading import load_engine
    kw.setdefault("max_tokens", 1024)
    return load_engine(folder, dtype=dtype, **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_long_decoding(folders, name, dtype):
    """7 prompt tokens, then 300 tokens one by one: five pages, every page edge crossed in decode."""
    cfg, seed = TINIES[name]
    toks = random_tokens(seed + 50, cfg["vocab_size"], 307)
    want = P.transformer_forward([toks], P.load_model_folder(folders[name]))[0]
    eng = load(folders[name], dtype)
    s = eng.open()
    got = [eng.step([(s, toks[:7], list(range(7)))])]
    for t in toks[7:]:
        got.append(eng.step([(s, [t], [0])]))
    got = torch.cat(got).double().cpu().numpy()
    errs = [rel_err(got[p], want[p]) for p in range(len(toks))]
    bad = [p for p, e in enumerate(errs) if e > TOL[dtype]]
    assert not bad, f"first wrong position {bad[0]} (page edge every 64), error {errs[bad[0]]:.3g}"
    assert eng.length(s) == 307
    eng.close(s)
    assert eng.cache.pages_in_use() == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_of_a_sequence(folders, dtype):
    """Prompts of one and two tokens (one token = no mask at all in the reference,
    crates/burn-lm-llama/src/nn/transformer.rs:169-171), then their first decoded tokens."""
    cfg, seed = TINIES["B"]
    plain = P.load_model_folder(folders["B"])
    eng = load(folders["B"], dtype)
    toks = random_tokens(3, cfg["vocab_size"], 6)
    want = P.transformer_forward([toks], plain)[0]
    a, b = eng.open(), eng.open()
    got = eng.step([(a, toks[:1], [0]), (b, toks[:2], [0, 1])]).double().cpu().numpy()
    for row, p in zip(got, [0, 0, 1]):
        assert rel_err(row, want[p]) <= TOL[dtype]
    got = eng.step([(a, [toks[1]], [0]), (b, [toks[2]], [0])]).double().cpu().numpy()
    assert rel_err(got[0], want[1]) <= TOL[dtype] and rel_err(got[1], want[2]) <= TOL[dtype]
    got = eng.step([(b, toks[3:6], [2]), (a, [toks[2]], [0])]).double().cpu().numpy()   # a chunk and a single token
    assert rel_err(got[0], want[5]) <= TOL[dtype] and rel_err(got[1], want[2]) <= TOL[dtype]


def test_a_far_key_among_hundreds_is_found(folders, tmp_path):
    """One early key is made to stand out for every later query, so an attention that loses keys far
    back, or a page of the table, changes the logits visibly.  In the first layer one lane of every
    head's query and key (lane 7, whose rotary pair turns by 0.13 rad over 400 positions) reads one
    feature of the normalised embedding; that feature is small and positive in every token's
    embedding and is all there is in the embedding of token 255, whose key therefore scores about
    e^6 against e^1 for every query."""
    from burn_lm_amd.weights import safetensors_io as st
    cfg, seed = TINIES["A"]
    f = st.open_folder(folders["A"])
    tensors = {n: f[n].tensor(n).clone() for n in f}
    j, lane, c = 5, 7, 2.0
    emb = tensors["model.embed_tokens.weight"].float()
    emb[:, j] = 0.1
    emb[255] = 0.0
    emb[255, j] = 1.0
    tensors["model.embed_tokens.weight"] = emb.bfloat16()
    for name, heads in (("q_proj", cfg["num_attention_heads"]), ("k_proj", cfg["num_key_value_heads"])):
        w = tensors[f"model.layers.0.self_attn.{name}.weight"].float()
        for h in range(heads):
            w[h * 16 + lane] = 0.0
            w[h * 16 + lane, j] = c
        tensors[f"model.layers.0.self_attn.{name}.weight"] = w.bfloat16()
    g = tensors["model.layers.0.input_layernorm.weight"].float()
    g[j] = 1.0
    tensors["model.layers.0.input_layernorm.weight"] = g.bfloat16()
    folder = str(tmp_path / "m")
    os.makedirs(folder)
    st.write_file(os.path.join(folder, "model.safetensors"), tensors.items())
    json.dump(cfg, open(os.path.join(folder, "config.json"), "w"))
    plain = P.load_model_folder(folder)
    toks = [t % 255 for t in random_tokens(11, 255, 400)]
    toks[3] = 255
    want = P.transformer_forward([toks], plain)[0]
    without = list(toks)
    without[3] = 7
    moved = P.transformer_forward([without], plain)[0]
    effect = [rel_err(moved[p], want[p]) for p in range(330, 400)]
    assert sum(e > 0.1 for e in effect) >= 60, "the test's own premise: the far key matters to the late positions"
    for dtype in ("float32", "bfloat16"):
        eng = load(folder, dtype)
        s = eng.open()
        eng.step([(s, toks[:330], [])])
        got = torch.cat([eng.step([(s, [t], [0])]) for t in toks[330:]]).double().cpu().numpy()
        for i, p in enumerate(range(330, 400)):
            assert rel_err(got[i], want[p]) <= TOL[dtype], f"{dtype}: position {p}"


def test_logits_do_not_depend_on_batch_mates_or_on_where_in_the_cache(folders):
    cfg, seed = TINIES["A"]
    eng = load(folders["A"], "float32", max_tokens=2048)
    toks = random_tokens(21, cfg["vocab_size"], 90)
    s = eng.open()
    alone = eng.step([(s, toks, list(range(90)))]).cpu()
    eng.close(s)
    # fill and free pages so that the same request lands on other pages and another slot
    junk = [eng.open() for _ in range(3)]
    eng.step([(j, random_tokens(30 + i, cfg["vocab_size"], 70 + 40 * i), []) for i, j in enumerate(junk)])
    eng.cache.views[0].k.fill_(float("nan"))   # what is left in pages must never be read
    eng.cache.views[1].v.fill_(float("nan"))
    for j in junk[:2]:
        eng.close(j)
    s = eng.open()
    other = eng.open()
    assert eng.cache.groups[0].tables[s] == []
    both = eng.step([(other, random_tokens(40, cfg["vocab_size"], 33), [32]), (s, toks, list(range(90)))]).cpu()
    assert torch.isfinite(both).all()
    assert rel_err(both[1:].double().numpy(), alone.double().numpy()) <= 2e-6


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(folders, name):
    """Unequal prompts, more requests than batch places, a stop token that ends one early: the
    32-bit engine gives the plain implementation's tokens."""
    from burn_lm_amd.server import InferenceServer
    cfg, seed = TINIES[name]
    plain = P.load_model_folder(folders[name])
    lens = [5, 11, 17, 1, 33, 7, 20]
    prompts = [random_tokens(60 + i, cfg["vocab_size"], n) for i, n in enumerate(lens)]
    free = [P.greedy_generate(plain, p, 10) for p in prompts]
    k = next((k for k in range(1, 10) if free[1][k] not in free[1][:k]), 0)   # a token request 1 makes first at place k
    stop = free[1][k]
    want = [P.greedy_generate(plain, p, 10, stop_ids=(stop,)) for p in prompts]
    server = InferenceServer(folders[name], dtype="float32", batch_size=3)
    server.config.update(max_seq_len=128, sample_len=10, temperature=0.0)
    results, stats = server.generate(prompts, stop_ids=[stop])
    assert [r.tokens for r in results] == want
    assert results[1].finish_reason == "stop" and len(results[1].tokens) == k + 1
    assert stats.generated_tokens == sum(len(w) for w in want) and stats.prompt_tokens == sum(lens)
    assert "Tokens Per Second" in stats.display_stats() and "##### BurnLM Stats" in stats.display_stats()
    # statelessness: the same request after others gives the same tokens (generate.rs:163-226)
    again, _ = server.generate([prompts[4]], stop_ids=[stop])
    assert again[0].tokens == want[4]
    assert server.engine.cache.pages_in_use() == 0


def test_temperature_sampling_is_seeded_and_independent_of_batch_mates(folders):
    from burn_lm_amd.server import InferenceServer
    cfg, seed = TINIES["B"]
    prompts = [random_tokens(80 + i, cfg["vocab_size"], n) for i, n in enumerate([1, 7, 20, 33])]
    server = InferenceServer(folders["B"], dtype="float32", batch_size=4)
    server.config.update(max_seq_len=128, sample_len=12, temperature=0.8, top_p=0.9, seed=11)
    a, _ = server.generate(prompts, stop_ids=[])
    b, _ = server.generate(prompts, stop_ids=[])
    assert [r.tokens for r in a] == [r.tokens for r in b]
    solo, _ = server.generate(prompts[:1], stop_ids=[])
    assert solo[0].tokens == a[0].tokens
    c, _ = server.generate(prompts, stop_ids=[], seed=12)
    assert [r.tokens for r in c] != [r.tokens for r in a]
    greedy, _ = server.generate(prompts, stop_ids=[], temperature=0.0)
    assert [r.tokens for r in greedy] != [r.tokens for r in a]


def test_a_refused_step_leaves_the_engine_as_it_was(folders):
    from burn_lm_amd.cache.cache import CacheFull, ContextOverflow
    from burn_lm_amd.engine.engine import StepError
    cfg, _ = TINIES["A"]
    eng = load(folders["A"], "float32", max_tokens=128)
    s = eng.open()
    eng.step([(s, [1, 2, 3], [])])
    for bad in ([(s, [], [])], [(s, [256], [0])], [(s, [1], [1])], [(s, [-1], [])], []):
        with pytest.raises(StepError):
            eng.step(bad)
    with pytest.raises((CacheFull, ContextOverflow)):
        eng.step([(s, [1] * 200, [])])
    t = eng.open()
    with pytest.raises(CacheFull):
        eng.step([(s, [1], [0]), (t, [1] * 100, [])])
    assert eng.length(s) == 3 and eng.length(t) == 0
    small = load(folders["A"], "float32", max_tokens=1024, max_context=64)
    u = small.open()
    with pytest.raises(ContextOverflow):
        small.step([(u, [1] * 65, [])])


def test_command_line_runs_a_prompt(folders, capsys):
    from burn_lm_amd.cli.main import main
    main(["-d", "f32", "run", folders["A"], "--sample-len", "6", "--tokens", "5,17,3"])
    out = capsys.readouterr().out
    plain = P.load_model_folder(folders["A"])
    assert ",".join(str(t) for t in P.greedy_generate(plain, [5, 17, 3], 6)) in out
    assert "##### BurnLM Stats" in out and "Tokens Per Second" in out
    main(["run", folders["A"], "--sample-len", "4", "--temperature", "0.7", "--seed", "3", "--no-stats", "hi"])
    assert "BurnLM Stats" not in capsys.readouterr().out
    # several prompts of unequal lengths: batches of two, one line per request, in the order given
    prompts = [[5, 17, 3], [9], [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11], [200, 100]]
    (tmp := os.path.join(folders["A"], "more.txt")) and open(tmp, "w").write("200 100\n")
    main(["-d", "f32", "run", folders["A"], "--sample-len", "5", "--tokens", "--batch", "2", "--no-stats", "--prompts-file", tmp]
         + [",".join(str(t) for t in p) for p in prompts[:3]])
    lines = [l for l in capsys.readouterr().out.splitlines() if l and l[0].isdigit()]
    assert lines == [",".join(str(t) for t in P.greedy_generate(plain, p, 5)) for p in prompts]
    main(["run", folders["A"], "--sample-len", "3", "--no-stats", "hi", "a longer prompt"])
    out = capsys.readouterr().out
    assert "[0] " in out and "[1] " in out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_replays_equal_eager_steps(folders, dtype):
    """Decode steps replayed from a captured graph against the same steps run eagerly on a second
    engine: several replays of one shape with eager work (prefills of other sequences, slot churn)
    and synchronisations between them, batches that shrink below their bucket (padding), and a page
    table that grows into the next width bucket."""
    cfg, seed = TINIES["A"]
    g = load(folders["A"], dtype, max_tokens=4096)
    e = load(folders["A"], dtype, max_tokens=4096, graphs=False)
    assert g.graphs.enabled and e.graphs is None
    lens = [3, 70, 130, 9, 40]
    prompts = [random_tokens(90 + i, cfg["vocab_size"], n) for i, n in enumerate(lens)]
    sg = [g.open() for _ in lens]
    se = [e.open() for _ in lens]
    a = g.step([(s, p, [len(p) - 1]) for s, p in zip(sg, prompts)])
    b = e.step([(s, p, [len(p) - 1]) for s, p in zip(se, prompts)])
    assert torch.equal(a, b)
    toks = [int(t) for t in a.argmax(1)]
    live = list(range(5))
    tol = 2e-6 if dtype == "float32" else 2e-2
    kept = []
    for k in range(400):
        a = g.step([(sg[i], [toks[i]], [0]) for i in live])
        b = e.step([(se[i], [toks[i]], [0]) for i in live])
        kept.append(a)
        assert rel_err(a.double().cpu().numpy(), b.double().cpu().numpy()) <= tol, f"decode step {k}, live {live}"
        for row, i in enumerate(live):
            toks[i] = int(b[row].argmax())
        if k == 5:                       # eager work between replays: another sequence is prefilled and dropped
            x = g.open(); g.step([(x, prompts[2], [])]); g.close(x)
            y = e.open(); e.step([(y, prompts[2], [])]); e.close(y)
            torch.cuda.synchronize()
        if k in (9, 30):                 # a sequence ends: 5 -> 4 -> 3 live in the bucket of 8 / 4 (the longest stays)
            i = live.pop(1 if k == 9 else 0)
            g.close(sg[i]); e.close(se[i])
    assert g.graphs.replays > 380 and len(g.graphs.captured) >= 3
    assert not torch.equal(kept[0], kept[1]), "each step's logits are a tensor of their own"
    assert max(g.length(sg[i]) for i in live) > 512, "the page table grew past the first width bucket"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_prompt_steps_replayed_from_graphs(folders, name, dtype):
    """Batches of unequal prompts one after another, slots used again: the first batch of a shape
    runs eagerly and is recorded, the later ones are replayed with padding sequences and padding
    tokens, with eager work and synchronisations between the replays.  Every prompt's last logits
    equal the plain implementation's, a prompt's second chunk on top of a replayed first one too,
    and so do the tokens decoded after a replayed prompt (they read the cache it wrote)."""
    cfg, seed = TINIES[name]
    plain = P.load_model_folder(folders[name])
    eng = load(folders[name], dtype, max_tokens=4096)
    V = cfg["vocab_size"]
    batches = [[40, 7, 90], [64, 1, 20, 33], [100, 3], [5, 5, 5, 120], [130], [61, 2, 70, 1], [150, 30], [128],
               [44, 9, 85], [60, 3, 66, 2], [129], [2, 50, 77]]      # a shape is recorded when it is met the second time
    seen_replay = 0
    for bi, lens in enumerate(batches):
        prompts = [random_tokens(1000 + 10 * bi + i, V, n + 3) for i, n in enumerate(lens)]
        want = [P.transformer_forward([p], plain)[0] for p in prompts]
        slots = [eng.open() for _ in lens]
        before = eng.graphs.replays
        got = eng.step([(s, p[:n], [n - 1]) for s, p, n in zip(slots, prompts, lens)]).double().cpu().numpy()
        seen_replay += eng.graphs.replays - before
        for i, n in enumerate(lens):
            assert rel_err(got[i], want[i][n - 1]) <= TOL[dtype], f"batch {bi} prompt {i} ({n} tokens)"
        if bi % 3 == 1:     # eager work between replays: a step that asks for every row cannot be replayed
            x = eng.open(); eng.step([(x, prompts[0][:9], list(range(9)))]); eng.close(x)
            torch.cuda.synchronize()
        # a second chunk of two tokens on top of the first, then one decoded token
        got = eng.step([(s, p[n:n + 2], [1]) for s, p, n in zip(slots, prompts, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            assert rel_err(got[i], want[i][n + 1]) <= TOL[dtype], f"batch {bi} prompt {i}: second chunk"
        got = eng.step([(s, [p[n + 2]], [0]) for s, p, n in zip(slots, prompts, lens)]).double().cpu().numpy()
        for i, n in enumerate(lens):
            assert rel_err(got[i], want[i][n + 2]) <= TOL[dtype], f"batch {bi} prompt {i}: decoded token"
        for s in slots:
            eng.close(s)
    assert eng.cache.pages_in_use() == 0
    prompt_shapes = [k for k in eng.graphs.captured if k[1] > 0]
    # whole prompts replayed (several batches have the shape of batch 0), and the second chunks
    assert seen_replay >= 2 and len(prompt_shapes) >= 4 and eng.graphs.replays >= 8, (seen_replay, sorted(eng.graphs.captured))


def test_a_part_that_is_not_graph_safe_turns_replay_off(folders):
    from burn_lm_amd.parts.attention import Attention
    eng = load(folders["A"], "float32")
    assert eng.graphs.enabled
    old = Attention.graph_safe
    Attention.graph_safe = False
    try:
        assert not load(folders["A"], "float32").graphs.enabled
    finally:
        Attention.graph_safe = old


def test_wide_layers_take_the_grouped_products(tmp_path):
    """A configuration wide enough (width 2048, feed-forward 4096) that the decode products of the
    output and down projections are cut over K into partial planes: prompts, then decoded tokens,
    against the plain implementation."""
    from burn_lm_amd.engine.runtime import Runtime
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=4096, num_hidden_layers=1,
               num_attention_heads=16, num_key_value_heads=4, head_dim=128, vocab_size=300, max_position_embeddings=256,
               rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False)
    rt = Runtime(torch.bfloat16, "cuda:0")
    assert rt.compute_units == 256
    # the fewest groups of at most 4096 of K whose blocks fill most of a round of the compute units
    assert rt.k_groups(2048, 2048) == 2 and rt.k_groups(2048, 4096) == 2 and rt.k_groups(6144, 2048) == 1
    assert rt.k_groups(2048, 8192) == 2 and rt.k_groups(16384, 2048) == 1 and rt.k_groups(4096, 4096) == 1
    assert rt.k_groups(3072, 3072) == 1 and rt.k_groups(3072, 8192) == 2 and rt.k_groups(4096, 14336) == 4
    assert rt.k_groups(2560, 11008) == 3 and rt.k_groups(96, 96) == 1 and rt.k_groups(2048, 100000) == 8
    assert rt.k_groups(2048, 8192, 40) == 4 and rt.k_groups(4096, 14336, 40) == 8     # more rows: shorter groups
    folder = make_folder(tmp_path / "wide", cfg, seed=5, std=0.03)
    plain = P.load_model_folder(folder)
    reqs = [random_tokens(200 + i, 300, n) for i, n in enumerate([20, 9, 41])]
    want = [P.transformer_forward([r], plain)[0] for r in reqs]
    eng = load(folder, "bfloat16", max_tokens=512)
    slots = [eng.open() for _ in reqs]
    cut = [len(r) - 6 for r in reqs]
    got = eng.step([(s, r[:c], [c - 1]) for s, r, c in zip(slots, reqs, cut)]).double().cpu().numpy()
    for i in range(3):
        assert rel_err(got[i], want[i][cut[i] - 1]) <= TOL["bfloat16"]
    for k in range(6):
        got = eng.step([(s, [r[c + k]], [0]) for s, r, c in zip(slots, reqs, cut)]).double().cpu().numpy()
        for i in range(3):
            assert rel_err(got[i], want[i][cut[i] + k]) <= TOL["bfloat16"], f"request {i}, decode step {k}"


@pytest.mark.parametrize("M,K,tile", [(33, 3072, (128, 128, 4)), (64, 2048, None), (65, 2048, (128, 128, 4)), (128, 520, (128, 128, 4)),
                                      (129, 2048, (256, 128)), (300, 4096, (256, 128)), (32, 3072, None)])
def test_float32_logits_of_many_rows_read_the_weights_once(monkeypatch, M, K, tile):
    """More rows than one skinny product takes at the width (more than 64, or more than 32 above K = 2048): the
    matrix-core kernel with a float32 output instead of the skinny product over chunks of rows."""
    from burn_lm_amd.csrc import ops
    from burn_lm_amd.engine.runtime import Runtime
    rt = Runtime(torch.bfloat16, "cuda:0")
    g = torch.Generator().manual_seed(M + K)
    N = 1000
    x = torch.randn(M, K, generator=g).bfloat16().cuda()
    raw = (torch.randn(N, K, generator=g) * 0.05).bfloat16().cuda()
    tiles, real = [], ops.gemm_mfma
    monkeypatch.setattr(ops, "gemm_mfma", lambda *a, **k: (tiles.append(k.get("tile")), real(*a, **k))[1])
    out = rt.linear(x, rt.weight(raw), out_dtype=torch.float32)
    assert tiles == ([tile] if tile else []) and out.dtype == torch.float32
    want = x.double() @ raw.double().T
    assert float((out.double() - want).abs().max() / want.abs().max()) < 2e-6


def test_short_prompts_take_the_fused_gate_up_product(tmp_path, monkeypatch):
    """Prompts of 65 rows and more whose gate/up tiles all run at once go through the matrix-core
    kernel with the gating in its epilogue (both of its deep-ring tiles), longer ones through the
    library product; the narrow products of short prompts come as partial planes over groups of K:
    all against the plain implementation."""
    from burn_lm_amd.csrc import ops
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=2048, intermediate_size=4096, num_hidden_layers=1,
               num_attention_heads=16, num_key_value_heads=4, head_dim=128, vocab_size=300, max_position_embeddings=2048,
               rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=False)
    folder = make_folder(tmp_path / "wide", cfg, seed=6, std=0.03)
    plain = P.load_model_folder(folder)
    tiles = []
    real = ops.gemm_mfma
    planes = []
    monkeypatch.setattr(ops, "gemm_mfma", lambda *a, **k: ((tiles if k.get("gated") else planes).append(k.get("tile")),
                                                           real(*a, **k))[1])
    rings, real_rows = [], ops.gemm_rows
    monkeypatch.setattr(ops, "gemm_rows", lambda a, w, out, **k: (rings.append(tuple(out.shape)), real_rows(a, w, out, **k))[1])
    fused_qkv, real_qkv = [], ops.gemm_rows_qkv_rope
    monkeypatch.setattr(ops, "gemm_rows_qkv_rope", lambda x, *a, **k: (fused_qkv.append(x.shape[0]), real_qkv(x, *a, **k))[1])
    eng = load(folder, "bfloat16", max_tokens=4096, graphs=False)
    # 70 rows: 128 blocks of the 128x64 tile; 100 + 150 rows: 256 of them; 300 + 90: 512, so the 128x128
    # tile with 256; 700 rows: 192 tiles of 256x128, one round on three quarters of the units; 600 rows fill
    # such tiles too little: the library; 2,000 rows: 256 tiles of 256x256
    for lengths, tile in (([70], (128, 64, 6)), ([100, 150], (128, 64, 6)), ([300, 90], (128, 128, 4)), ([700], (256, 128)),
                          ([600], None), ([1500, 500], (256, 256))):
        reqs = [random_tokens(300 + i + sum(lengths), 300, n) for i, n in enumerate(lengths)]
        want = [P.transformer_forward([r], plain)[0] for r in reqs]
        slots = [eng.open() for _ in reqs]
        del tiles[:], planes[:], rings[:], fused_qkv[:]
        got = eng.step([(s, r, [0, len(r) // 2, len(r) - 1]) for s, r in zip(slots, reqs)]).double().cpu().numpy()
        assert tiles == ([tile] if tile else []), (lengths, tiles)
        # up to 256 rows the output projection (K = 2048) runs on the product of 17 to 64 rows with a block for
        # every 64 rows: two partial planes while that leaves every block a compute unit, else one result; the
        # q/k/v projection with the rotation too (32 columns per block, 64 where those would be too many blocks)
        M = sum(lengths)
        assert rings == ([(2, M, 2048)] if M <= 128 else [(M, 2048)] if M <= 256 else []), (lengths, rings)
        assert fused_qkv == ([M] if M <= 256 else []), (lengths, fused_qkv)
        # the other narrow products come as partial planes where a few groups of K fill the chip
        n_planes = sum(1 for N, K in ((2048, 2048), (2048, 4096))
                       if not eng.rt.mid_rows_ring(M, N, K, True) and eng.rt.mid_k_groups(M, N, K))
        assert len(planes) == n_planes and (n_planes >= 1) == (M <= 512), (lengths, planes)
        for i, r in enumerate(reqs):
            for j, pos in enumerate([0, len(r) // 2, len(r) - 1]):
                assert rel_err(got[3 * i + j], want[i][pos]) <= TOL["bfloat16"], (lengths, i, pos)
        for s in slots:
            eng.close(s)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("n,bucket", [(20, 24), (70, 96)])
def test_graph_replays_of_larger_batches(folders, dtype, n, bucket):
    """20 sequences per decode step: the skinny product with several row tiles; 70: the layer products
    are the library's, recorded into the graph.  Every replay is checked against the eager engine,
    with eager prefills and synchronisations between replays."""
    cfg, seed = TINIES["B"]
    g = load(folders["B"], dtype, max_tokens=16384, max_seqs=80)
    e = load(folders["B"], dtype, max_tokens=16384, max_seqs=80, graphs=False)
    prompts = [random_tokens(300 + i, cfg["vocab_size"], 3 + (7 * i) % 40) for i in range(n)]
    sg = [g.open() for _ in range(n)]
    se = [e.open() for _ in range(n)]
    a = g.step([(s, p, [len(p) - 1]) for s, p in zip(sg, prompts)])
    b = e.step([(s, p, [len(p) - 1]) for s, p in zip(se, prompts)])
    toks = [int(t) for t in b.argmax(1)]
    tol = 2e-6 if dtype == "float32" else 2e-2
    live = list(range(n))
    for k in range(40):
        a = g.step([(sg[i], [toks[i]], [0]) for i in live])
        b = e.step([(se[i], [toks[i]], [0]) for i in live])
        assert rel_err(a.double().cpu().numpy(), b.double().cpu().numpy()) <= tol, f"decode step {k}"
        for row, i in enumerate(live):
            toks[i] = int(b[row].argmax())
        if k % 9 == 4:          # eager work between replays, and the batch shrinks within its bucket
            x = g.open(); g.step([(x, prompts[0], [])]); g.close(x)
            y = e.open(); e.step([(y, prompts[0], [])]); e.close(y)
            i = live.pop(3)
            g.close(sg[i]); e.close(se[i])
            torch.cuda.synchronize()
    assert g.graphs.replays >= 35 and any(k[0] == bucket for k in g.graphs.captured)


def test_head_size_that_is_no_power_of_two_and_odd_counts(tmp_path):
    """head_dim 48 (a step of 16 that is no power of two), 5 heads without grouping, an odd
    vocabulary: whole, tail and batch against plain."""
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=120, intermediate_size=200, num_hidden_layers=2,
               num_attention_heads=5, num_key_value_heads=5, head_dim=48, vocab_size=257, max_position_embeddings=256,
               rms_norm_eps=1e-5, rope_theta=10000.0, tie_word_embeddings=True)
    folder = make_folder(tmp_path / "m48", cfg, seed=9)
    plain = P.load_model_folder(folder)
    reqs = [random_tokens(400 + i, 257, n) for i, n in enumerate([70, 5, 130])]
    want = [P.transformer_forward([r], plain)[0] for r in reqs]
    for dtype in ("float32", "bfloat16"):
        eng = load(folder, dtype, max_tokens=1024)
        slots = [eng.open() for _ in reqs]
        cut = [len(r) - 4 for r in reqs]
        got = eng.step([(s, r[:c], list(range(c))) for s, r, c in zip(slots, reqs, cut)]).double().cpu().numpy()
        o = 0
        for r, c, w in zip(reqs, cut, want):
            assert rel_err(got[o:o + c], w[:c]) <= TOL[dtype], dtype
            o += c
        for k in range(4):
            got = eng.step([(s, [r[c + k]], [0]) for s, r, c in zip(slots, reqs, cut)]).double().cpu().numpy()
            for i in range(3):
                assert rel_err(got[i], want[i][cut[i] + k]) <= TOL[dtype], f"{dtype} request {i} decode {k}"


def _write_folder(path, cfg, tensors):
    from burn_lm_amd.weights import safetensors_io as st
    os.makedirs(path, exist_ok=True)
    json.dump(cfg, open(os.path.join(path, "config.json"), "w"))
    st.write_file(os.path.join(path, "model.safetensors"), tensors.items())
    return str(path)


def test_the_references_whole_model_vector_in_32_bit(tmp_path):
    """crates/burn-lm-llama/src/nn/transformer.rs:299-349: vocabulary 8, 2 layers, width 8, inner 16,
    2 heads on 1 KV head (head_dim 4), every tensor arange(n)*5/n in the reference's [d_in, d_out]
    order (the Range initialiser of the random-weights mode, whose tensors tests/test_weights.py checks),
    token ids [[0, 1], [2, 3]].  The engine reads them as a Meta-named 32-bit checkpoint and must give
    the reference's logits."""
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=8, intermediate_size=16, num_hidden_layers=2,
               num_attention_heads=2, num_key_value_heads=1, vocab_size=8, rms_norm_eps=1e-5, rope_theta=10000.0,
               tie_word_embeddings=False, max_position_embeddings=64)
    want = np.array([[[56.37573, 57.77283, 59.169933, 60.567043, 61.964146, 63.361248, 64.758354, 66.15546],
                      [56.374626, 57.77171, 59.168793, 60.56588, 61.962963, 63.360046, 64.75713, 66.15422]],
                     [[56.374252, 57.771328, 59.168407, 60.565487, 61.962566, 63.359642, 64.75672, 66.1538],
                      [56.37408, 57.771156, 59.168232, 60.565304, 61.96238, 63.359455, 64.75653, 66.15361]]])
    import burn_lm_amd
    from burn_lm_amd.weights.random_init import Range
    folder = burn_lm_amd.write_random_model(str(tmp_path / "ref"), cfg, init=Range(0.0, 5.0), names="meta", dtype=torch.float32)
    eng = load(folder, "float32")
    a, b = eng.open(), eng.open()
    got = eng.step([(a, [0, 1], [0, 1]), (b, [2, 3], [0, 1])]).double().cpu().numpy().reshape(2, 2, 8)
    np.testing.assert_allclose(got, want, rtol=2e-6)
    # the same, token by token from the cache
    eng.close(a); eng.close(b)
    a = eng.open()
    one = [eng.step([(a, [tok], [0])]).double().cpu().numpy()[0] for tok in (0, 1)]
    np.testing.assert_allclose(np.stack(one), want[0], rtol=2e-6)


def test_meta_names_equal_hugging_face_names_and_a_tied_head_equals_a_copied_one(folders, tmp_path):
    """The same model under the two checkpoint layouts (import.rs:20-88): Meta names with the q/k rows
    in adjacent-pair order (import.rs:94-127) against Hugging Face names with half-split rows; and
    tie_word_embeddings against an lm_head that is a copy of the table."""
    from burn_lm_amd.models.llama import HF_NAMES, META_NAMES
    from burn_lm_amd.weights import safetensors_io as st
    cfg = dict(TINY_A)
    f = st.open_folder(folders["A"])
    hf = {name: file.tensor(name).clone() for name, file in f.items()}
    meta = {}
    for name, w in hf.items():
        new = name.replace(HF_NAMES["embedding"], META_NAMES["embedding"]).replace(HF_NAMES["final_norm"], META_NAMES["final_norm"])
        new = new.replace("model.layers.", "layers.")
        for key in ("q", "k", "v", "o", "gate", "up", "down", "mixer_norm", "ffn_norm"):
            new = new.replace(HF_NAMES[key], META_NAMES[key])
        if name.endswith(HF_NAMES["q"]) or name.endswith(HF_NAMES["k"]):
            heads = cfg["num_attention_heads"] if name.endswith(HF_NAMES["q"]) else cfg["num_key_value_heads"]
            w = torch.from_numpy(P.permute_hf_rows(w.float().numpy(), heads).copy()).to(w.dtype)
        meta[new] = w
    assert "tok_embeddings.weight" in meta and "layers.1.attention.wq.weight" in meta
    untied = dict(hf); untied["lm_head.weight"] = hf[HF_NAMES["embedding"]].clone()
    toks = [random_tokens(500 + i, cfg["vocab_size"], n) for i, n in enumerate([40, 9])]
    outs = {}
    for key, c, t in (("hf", cfg, hf), ("meta", cfg, meta), ("untied", dict(cfg, tie_word_embeddings=False), untied)):
        eng = load(_write_folder(tmp_path / key, c, t), "float32")
        slots = [eng.open() for _ in toks]
        outs[key] = eng.step([(s, tk, list(range(len(tk)))) for s, tk in zip(slots, toks)]).double().cpu().numpy()
    assert rel_err(outs["meta"], outs["hf"]) <= 2e-6
    assert np.array_equal(outs["untied"], outs["hf"])


def test_sampled_tokens_follow_the_plain_probabilities(folders):
    """Prompts of 1, 7, 20 and 33 tokens, 12 tokens each at temperature 0.8 and top-p 0.9 in 32-bit:
    every token the engine draws lies in the plain implementation's nucleus, and its interval of
    the plain cumulative distribution (kept tokens in index order) holds the draw's uniform number."""
    from burn_lm_amd.sampling.sampler import uniform
    from burn_lm_amd.server import InferenceServer
    cfg, seed = TINIES["B"]
    plain = P.load_model_folder(folders["B"])
    prompts = [random_tokens(80 + i, cfg["vocab_size"], n) for i, n in enumerate([1, 7, 20, 33])]
    server = InferenceServer(folders["B"], dtype="float32", batch_size=4)
    server.config.update(max_seq_len=128, sample_len=12, temperature=0.8, top_p=0.9, seed=11)
    results, _ = server.generate(prompts, stop_ids=[])
    for i, res in enumerate(results):
        seq = list(prompts[i])
        assert len(res.tokens) == 12
        for n, tok in enumerate(res.tokens):
            probs = P.temperature_softmax(P.transformer_forward([seq], plain)[0][-1], 0.8)
            kept = sorted(P.top_p_keep(probs, 0.9))
            assert tok in kept, f"request {i} token {n}"
            cdf = np.cumsum(probs[kept]) / probs[kept].sum()
            k = kept.index(tok)
            u = uniform(11, i, n)
            assert (cdf[k - 1] if k else 0.0) - 1e-4 <= u <= cdf[k] + 1e-4, f"request {i} token {n}"
            seq.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_fed_in_uneven_chunks_beside_a_decoding_neighbour(folders, dtype):
    """Any cut of a sequence into steps gives the same logits: a 300-token prompt in chunks of 100, 28,
    64, 1, 90 and 17 tokens (chunk ends on, before and after page edges), while a second sequence in
    the same steps goes on one token at a time."""
    cfg, seed = TINIES["A"]
    plain = P.load_model_folder(folders["A"])
    eng = load(folders["A"], dtype, max_tokens=2048)
    long_req = random_tokens(700, cfg["vocab_size"], 300)
    short = random_tokens(701, cfg["vocab_size"], 40)
    want_long = P.transformer_forward([long_req], plain)[0]
    want_short = P.transformer_forward([short], plain)[0]
    a, b = eng.open(), eng.open()
    got = eng.step([(b, short[:34], [33])]).double().cpu().numpy()
    assert rel_err(got[0], want_short[33]) <= TOL[dtype]
    at, k = 0, 34
    for n in (100, 28, 64, 1, 90, 17):
        rows = sorted({0, n // 2, n - 1})
        got = eng.step([(a, long_req[at:at + n], rows), (b, [short[k]], [0])]).double().cpu().numpy()
        for j, r in enumerate(rows):
            assert rel_err(got[j], want_long[at + r]) <= TOL[dtype], f"{dtype} chunk at {at} row {r}"
        assert rel_err(got[len(rows)], want_short[k]) <= TOL[dtype], f"{dtype} neighbour at {k}"
        at += n
        k += 1
    assert at == 300


@pytest.mark.parametrize("name,dtype,seed", [("A", "float32", 0), ("B", "float32", 1), ("A", "bfloat16", 2), ("B", "bfloat16", 3),
                                             ("C", "float32", 4), ("C", "bfloat16", 5)])
def test_random_schedules_of_steps(folders, name, dtype, seed):
    """Sequences are opened, fed in random chunks (whole prompts, pieces, single tokens, several
    sequences per step in random order), and closed at random, on a cache small enough that slots and
    pages are used again and steps are sometimes refused; every logit asked for is compared with the
    plain implementation's for that sequence and position."""
    from burn_lm_amd.cache.cache import CacheFull
    cfg, _ = TINIES[name]
    plain = P.load_model_folder(folders[name])
    rng = np.random.default_rng(100 + seed)
    max_ctx = min(cfg["max_position_embeddings"], 256)
    eng = load(folders[name], dtype, max_tokens=768, max_seqs=5, max_context=max_ctx)
    live = {}        # slot -> [tokens of the sequence, fed so far, plain logits]
    checked = refused = 0
    for it in range(60):
        if len(live) < 5 and (not live or rng.random() < 0.5):
            try:
                s = eng.open()
            except CacheFull:
                s = None
            if s is not None:
                toks = random_tokens(int(rng.integers(1 << 30)), cfg["vocab_size"], int(rng.integers(1, 200)))
                live[s] = [toks, 0, P.transformer_forward([toks], plain)[0]]
        picks = [s for s in live if rng.random() < 0.7]
        rng.shuffle(picks)
        entries, expect = [], []
        for s in picks:
            toks, fed, want = live[s]
            left = len(toks) - fed
            if left == 0:
                continue
            n = int(min(left, rng.choice([1, 1, 2, 17, 64, 65, 200])))
            rows = sorted(set(int(r) for r in rng.integers(0, n, size=int(rng.integers(0, 4)))))
            entries.append((s, toks[fed:fed + n], rows))
            expect += [want[fed + r] for r in rows]
        if entries:
            try:
                got = eng.step(entries)
            except CacheFull:
                refused += 1
                got = None
                victim = max(live, key=lambda s: live[s][1])     # make room: the longest sequence goes
                eng.close(victim)
                del live[victim]
                entries = []
            for s, t, _ in entries:
                live[s][1] += len(t)
            if got is not None:
                got = got.double().cpu().numpy()
                assert got.shape[0] == len(expect)
                for g_row, w_row in zip(got, expect):
                    assert rel_err(g_row, w_row) <= TOL[dtype], f"iteration {it}"
                    checked += 1
            elif entries:
                assert not expect
        for s in list(live):
            if live[s][1] == len(live[s][0]) or rng.random() < 0.05:
                eng.close(s)
                del live[s]
    assert checked > 60, f"only {checked} logits were compared"
    for s in list(live):
        eng.close(s)
    assert eng.cache.pages_in_use() == 0 and eng.cache.free_slots == 5


@pytest.mark.parametrize("name,dtype,seed", [("A", "bfloat16", 0), ("B", "float32", 1), ("C", "bfloat16", 2)])
def test_random_schedules_through_recorded_graphs(folders, name, dtype, seed):
    """Like the random schedules above, but every step asks for the last logits of each of its
    sequences, so decode steps and prompt steps (whole prompts, pieces, mixed with single tokens)
    run from recorded graphs as soon as their shape has been seen: slots and pages are used
    again, shapes alternate, and every logit is compared with the plain implementation's."""
    from burn_lm_amd.cache.cache import CacheFull
    cfg, _ = TINIES[name]
    plain = P.load_model_folder(folders[name])
    rng = np.random.default_rng(1000 + seed)
    eng = load(folders[name], dtype, max_tokens=1024, max_seqs=6, max_context=min(cfg["max_position_embeddings"], 256))
    live, checked = {}, 0
    for it in range(160):
        if len(live) < 6 and (not live or rng.random() < 0.5):
            try:
                s = eng.open()
            except CacheFull:
                s = None
            if s is not None:
                toks = random_tokens(int(rng.integers(1 << 30)), cfg["vocab_size"], int(rng.integers(1, 200)))
                live[s] = [toks, 0, P.transformer_forward([toks], plain)[0]]
        picks = [s for s in live if rng.random() < 0.7]
        rng.shuffle(picks)
        single = rng.random() < 0.5
        entries, expect = [], []
        for s in picks:
            toks, fed, want = live[s]
            if fed == len(toks):
                continue
            n = 1 if single else int(min(len(toks) - fed, rng.choice([1, 2, 17, 64, 65, 130])))
            entries.append((s, toks[fed:fed + n], [n - 1]))
            expect.append(want[fed + n - 1])
        if entries:
            try:
                got = eng.step(entries).double().cpu().numpy()
            except CacheFull:
                victim = max(live, key=lambda s: live[s][1])
                eng.close(victim)
                del live[victim]
                continue
            for s, t, _ in entries:
                live[s][1] += len(t)
            for g_row, w_row in zip(got, expect):
                assert rel_err(g_row, w_row) <= TOL[dtype], f"iteration {it}"
                checked += 1
        for s in list(live):
            if live[s][1] == len(live[s][0]) or rng.random() < 0.05:
                eng.close(s)
                del live[s]
    for s in list(live):
        eng.close(s)
    assert eng.cache.pages_in_use() == 0
    shapes = eng.graphs.captured
    assert checked > 200 and eng.graphs.replays > 60 and any(k[1] > 0 for k in shapes) and any(k[1] == 0 for k in shapes)



@pytest.mark.parametrize("name,layers,vocab", [("llama3.2-1b", 2, None), ("llama3.2-3b", 1, 20008), ("llama3.1-8b", 1, 20008)])
def test_the_benchmark_layer_shapes_against_the_plain_implementation(tmp_path, name, layers, vocab):
    """Layers of the shapes that the measurements are quoted on, at which the products' policies choose
    differently than at the small configurations.  Llama-3.2-1B (two layers, whole vocabulary of
    128,256, tied head): width 2048, 32 heads in 8 groups, feed-forward 8192: K-groups, the fused
    gate/up product in whole rounds of tiles, the head over the whole vocabulary.  Llama-3.2-3B: width
    3072, 24 heads of size 128 in groups of 3.  Llama-3.1-8B: width 4096, feed-forward 14336, separate
    head: long K in the down projection, the library's products above 32 rows.  (The two wide shapes
    with one layer and a vocabulary of 20,008, which is no multiple of 16: their layers are what
    differs.)  Prompts of 2,048, 700 and 76 tokens alone and in one batch, then twelve tokens one by
    one at batch 1 and 3; then the three among 37 shorter prompts, a batch of 40, and twelve tokens
    each; in both dtypes."""
    from burn_lm_amd.config.presets import preset
    cfg = dict(preset(name))
    cfg["num_hidden_layers"] = layers
    if vocab:
        cfg["vocab_size"] = vocab
        cfg.pop("eos_token_id", None), cfg.pop("bos_token_id", None)     # they lie beyond the smaller vocabulary
    folder = make_folder(tmp_path / "shape", cfg, seed=3, std=0.02)
    plain = P.load_model_folder(folder)
    n_dec = 12
    lengths = [2048, 700, 76] + [1 + (29 * i) % 150 for i in range(37)]
    reqs = [random_tokens(40 + i, cfg["vocab_size"], n + n_dec) for i, n in enumerate(lengths)]

    def plain_rows(toks, rows):   # the plain blocks, with the head on the wanted rows only
        h = plain["tok_embeddings"][np.asarray([toks])]
        for lw in plain["layers"]:
            h = P.block(h, lw, plain["cfg"], plain["freqs"], 0)
        return P.rms_norm(h, plain["norm"], plain["cfg"]["eps"])[0][rows] @ plain["output"].T

    want = []
    for r in reqs:
        cut = len(r) - n_dec
        want.append(plain_rows(r, [0, cut // 2, cut - 1] + list(range(cut, len(r)))))
    for dtype, tol in (("float32", 1e-5), ("bfloat16", TOL["bfloat16"])):
        eng = load(folder, dtype, max_tokens=2176 + 832 + 128 + 37 * 192, max_seqs=40)
        for group in ([0], [1], [2], [0, 1, 2], list(range(40))):
            slots = {i: eng.open() for i in group}
            cut = {i: len(reqs[i]) - n_dec for i in group}
            got = eng.step([(slots[i], reqs[i][:cut[i]], [0, cut[i] // 2, cut[i] - 1]) for i in group]).double().cpu().numpy()
            for k, i in enumerate(group):
                for j in range(3):
                    assert rel_err(got[3 * k + j], want[i][j]) <= tol, f"{dtype} batch of {len(group)}: request {i}, prompt row {j}"
            for s in range(n_dec):
                got = eng.step([(slots[i], [reqs[i][cut[i] + s]], [0]) for i in group]).double().cpu().numpy()
                for k, i in enumerate(group):
                    assert rel_err(got[k], want[i][3 + s]) <= tol, f"{dtype} batch of {len(group)}: request {i}, decode step {s}"
            for i in group:
                eng.close(slots[i])
        del eng
        torch.cuda.empty_cache()


def test_wanted_places_come_back_in_the_order_given(folders):
    """Logits come in the order of the entries and, within an entry, of its list of wanted places as
    given: unsorted, and with a place named twice."""
    cfg, seed = TINIES["A"]
    plain = P.load_model_folder(folders["A"])
    a, b = random_tokens(810, cfg["vocab_size"], 9), random_tokens(811, cfg["vocab_size"], 5)
    wa, wb = P.transformer_forward([a], plain)[0], P.transformer_forward([b], plain)[0]
    eng = load(folders["A"], "float32")
    sa, sb = eng.open(), eng.open()
    got = eng.step([(sa, a, [7, 0, 7, 3]), (sb, b, [4, 1])]).double().cpu().numpy()
    assert got.shape[0] == 6
    for row, want in zip(got, [wa[7], wa[0], wa[7], wa[3], wb[4], wb[1]]):
        assert rel_err(row, want) <= TOL["float32"]


def test_checkpoints_stored_in_32_bit_and_in_float16(tmp_path, capsys):
    """The same random model stored as float32, as bfloat16 and as float16.  A tensor stored in 32 bits
    stays in 32 bits in a bfloat16 run (its products then run on the float kernels, and a note says so),
    unless the loader is asked to round matrices to the run's type, which gives the very engine of the
    bfloat16 folder.  Float16 is rounded to bfloat16 (three bits of each weight): the run then equals
    the plain implementation *of the rounded weights* within the usual tolerance, and the stored ones
    within 6 % of the largest logit; a float32 run of it is exact."""
    cfg, seed = TINIES["C"]
    toks = random_tokens(900, cfg["vocab_size"], 150)
    f32 = make_folder(tmp_path / "f32", cfg, seed, dtype=torch.float32)
    b16 = make_folder(tmp_path / "b16", cfg, seed, dtype=torch.bfloat16)
    f16 = make_folder(tmp_path / "f16", cfg, seed, dtype=torch.float16)

    def run(folder, dtype, **kw):
        eng = load(folder, dtype, **kw)
        s = eng.open()
        whole = eng.step([(s, toks[:140], list(range(140)))]).double().cpu().numpy()
        tail = [eng.step([(s, [t], [0])]).double().cpu().numpy()[0] for t in toks[140:]]
        return eng, np.concatenate([whole, np.stack(tail)])

    # stored in 32 bits, bfloat16 run: the matrices stay float32, and the run says so
    want32 = P.transformer_forward([toks], P.load_model_folder(f32))[0]
    capsys.readouterr()
    eng, got = run(f32, "bfloat16")
    note = capsys.readouterr().err
    assert "stored in 32 bits" in note and "cast_32bit" in note
    assert eng.model.blocks[0].mixer.w_qkv.dtype == torch.float32 and not eng.model.blocks[0].mixer.w_qkv.packable
    assert max(rel_err(got[p], want32[p]) for p in range(150)) <= TOL["bfloat16"]
    # the same folder with its matrices rounded when they are loaded: the packed products, and the
    # bfloat16 folder's logits to the bit (the weights are the same bytes then; norm weights stay wide)
    eng_c, got_c = run(f32, "bfloat16", cast_32bit=True)
    assert eng_c.model.blocks[0].mixer.w_qkv.dtype == torch.bfloat16 and eng_c.model.blocks[0].mixer.w_qkv.packable
    assert eng_c.model.blocks[0].mixer_norm.gamma.dtype == torch.float32
    plain16 = P.load_model_folder(b16)
    want16 = P.transformer_forward([toks], plain16)[0]
    assert max(rel_err(got_c[p], want16[p]) for p in range(150)) <= TOL["bfloat16"]
    # float32 run of the float32 folder
    _, got = run(f32, "float32")
    assert max(rel_err(got[p], want32[p]) for p in range(150)) <= TOL["float32"]
    # float16: exact in a float32 run; rounded to bfloat16 in a bfloat16 run
    plain_h = P.load_model_folder(f16)
    want_h = P.transformer_forward([toks], plain_h)[0]
    _, got = run(f16, "float32")
    assert max(rel_err(got[p], want_h[p]) for p in range(150)) <= TOL["float32"]
    rounded = dict(plain_h, tok_embeddings=P.round_bf16(plain_h["tok_embeddings"]), norm=P.round_bf16(plain_h["norm"]),
                   layers=[{k: P.round_bf16(v) for k, v in lw.items()} for lw in plain_h["layers"]])
    rounded["output"] = rounded["tok_embeddings"]     # config C ties its head
    want_r = P.transformer_forward([toks], rounded)[0]
    eng_h, got = run(f16, "bfloat16")
    assert eng_h.model.blocks[0].mixer.w_qkv.dtype == torch.bfloat16
    assert max(rel_err(got[p], want_r[p]) for p in range(150)) <= TOL["bfloat16"]
    assert max(rel_err(got[p], want_h[p]) for p in range(150)) <= 6e-2


@pytest.mark.parametrize("name", ["A", "C"])
def test_generation_that_runs_ahead_of_the_host_in_bfloat16(folders, name):
    """The generation loop keeps the picked tokens on the GPU and starts the next step from them
    before the host has seen them (step_ahead and pick_device, from recorded graphs).  In bfloat16, on
    the matrix-core paths, it must give the tokens of the plain loop that reads every token first
    (an engine shown without step_ahead), and the logits behind the first tokens must be the plain
    implementation's within the tolerance."""
    from burn_lm_amd.engine.generate import generate
    from burn_lm_amd.sampling.sampler import Sampler
    cfg, seed = TINIES[name]
    eng = load(folders[name], "bfloat16", max_tokens=4096, max_seqs=8)
    prompts = [random_tokens(700 + i, cfg["vocab_size"], n) for i, n in enumerate([5, 70, 17, 1, 33, 130, 9])]

    class Plain:      # the same engine without the run-ahead entry: the loop then waits for every token
        def __init__(self, e):
            self.open, self.close, self.step, self.length = e.open, e.close, e.step, e.length
            self.max_context, self.cache = e.max_context, e.cache

    stop = 3
    for temperature, top_p in ((0.0, 1.0), (0.7, 0.9)):
        for _ in range(2):          # the second round replays what the first recorded
            ahead, stats = generate(eng, prompts, Sampler(temperature, top_p, seed=5), 24, stop_ids=[stop], batch_size=4)
            waited, _ = generate(Plain(eng), prompts, Sampler(temperature, top_p, seed=5), 24, stop_ids=[stop], batch_size=4)
            assert [r.tokens for r in ahead] == [r.tokens for r in waited]
            assert [r.finish_reason for r in ahead] == [r.finish_reason for r in waited]
    assert eng.graphs.replays > 40 and eng.cache.pages_in_use() == 0
    # the logits behind the first generated token of each request, against the plain implementation
    plain = P.load_model_folder(folders[name])
    for p in prompts:
        s = eng.open()
        got = eng.step([(s, p, [len(p) - 1])]).double().cpu().numpy()[0]
        eng.close(s)
        assert rel_err(got, P.transformer_forward([p], plain)[0, -1]) <= TOL["bfloat16"]


def test_run_ahead_with_an_embedding_that_cannot_take_tokens_from_the_device(folders):
    """An embedding part without forward_from (here: the framework's own with the method hidden) gets the
    picked tokens gathered into the step's token ids by a launch in front of the replay; generation
    gives the same tokens as the loop that reads every token first."""
    from burn_lm_amd.engine.generate import generate
    from burn_lm_amd.parts.embedding import Embedding
    from burn_lm_amd.sampling.sampler import Sampler
    cfg, seed = TINIES["B"]

    class PlainEmbedding(Embedding):
        def __getattribute__(self, name):
            if name == "forward_from":
                raise AttributeError(name)
            return super().__getattribute__(name)

    eng = load(folders["B"], "bfloat16", max_tokens=2048, max_seqs=4)
    eng.model.embedding.__class__ = PlainEmbedding
    assert not hasattr(eng.model.embedding, "forward_from")
    prompts = [random_tokens(40 + i, cfg["vocab_size"], n) for i, n in enumerate([9, 33, 2])]

    class Waiting:
        def __init__(self, e):
            self.open, self.close, self.step, self.length = e.open, e.close, e.step, e.length
            self.max_context, self.cache = e.max_context, e.cache

    for _ in range(2):
        ahead, _ = generate(eng, prompts, Sampler(0.0), 20, stop_ids=[], batch_size=4)
        waited, _ = generate(Waiting(eng), prompts, Sampler(0.0), 20, stop_ids=[], batch_size=4)
        assert [r.tokens for r in ahead] == [r.tokens for r in waited]
    assert eng.graphs.replays > 20
    assert all(not c.folded for c in eng.graphs.captured.values())


def test_recorded_shapes_are_limited_and_the_oldest_goes(folders, monkeypatch):
    """A shape is recorded at its second sight; with room for two recorded shapes a third one evicts
    the shape replayed longest ago, and every step still gives the plain logits."""
    from burn_lm_amd.engine import graphs
    monkeypatch.setattr(graphs, "MAX_GRAPHS", 2)
    cfg, seed = TINIES["A"]
    plain = P.load_model_folder(folders["A"])
    eng = load(folders["A"], "float32", max_tokens=4096, max_seqs=16)
    seqs = [random_tokens(990 + i, cfg["vocab_size"], 30) for i in range(9)]
    want = [P.transformer_forward([t], plain)[0] for t in seqs]
    slots = [eng.open() for _ in seqs]
    eng.step([(s, t[:4], []) for s, t in zip(slots, seqs)])
    recorded_after = {}
    for p in range(4, 30):
        n = (1, 2, 3, 5, 9)[(p // 5) % 5]         # live sequences this step: buckets 1, 2, 4, 8, 16
        live = list(range(9)) if p % 5 == 0 else list(range(n))
        # every sequence must advance together, so the idle ones take the same step in a second call
        got = eng.step([(slots[i], [seqs[i][p]], [0]) for i in live]).double().cpu().numpy()
        for k, i in enumerate(live):
            assert rel_err(got[k], want[i][p]) <= TOL["float32"], (p, i)
        rest = [i for i in range(9) if i not in live]
        if rest:
            eng.step([(slots[i], [seqs[i][p]], []) for i in rest])
        recorded_after[p] = len(eng.graphs.captured)
    assert max(recorded_after.values()) <= 2 and eng.graphs.evicted >= 1 and eng.graphs.replays >= 4


def test_random_weights_are_the_same_bytes_on_the_gpu_and_in_a_folder(tmp_path):
    """An engine with random weights made on the GPU is the engine loaded from the folder that the
    random-weights mode writes on the CPU for the same configuration and seed: the tensors are equal
    to the byte, so the logits are equal to the bit."""
    from burn_lm_amd import registry
    from burn_lm_amd.engine.loading import random_engine
    from burn_lm_amd.weights.random_init import random_tensors
    cfg, _ = TINIES["B"]
    arch = registry.architecture_of(cfg)
    on_cpu = dict(random_tensors(arch, arch.read_config(cfg), 21, std=0.08, norm_jitter=0.1))
    on_gpu = dict(random_tensors(arch, arch.read_config(cfg), 21, std=0.08, norm_jitter=0.1, device="cuda"))
    assert list(on_cpu) == list(on_gpu)
    for n in on_cpu:
        assert on_gpu[n].is_cuda and torch.equal(on_cpu[n], on_gpu[n].cpu()), n
    folder = make_folder(tmp_path / "m", cfg, 21)
    toks = random_tokens(77, cfg["vocab_size"], 40)
    for dtype in ("float32", "bfloat16"):
        a = load(folder, dtype)
        b = random_engine(cfg, seed=21, dtype=dtype, max_tokens=1024, std=0.08, norm_jitter=0.1)
        sa, sb = a.open(), b.open()
        assert torch.equal(a.step([(sa, toks, list(range(40)))]), b.step([(sb, toks, list(range(40)))]))


def test_prompts_fed_within_a_budget_give_the_tokens_of_one_step(folders):
    """generate() with a prompt budget smaller than a batch's prompts feeds them in several steps (prompts cut
    where a step is full); in 32-bit the tokens equal those of the run that feeds each batch in one step,
    and the plain implementation's."""
    from burn_lm_amd.engine.generate import generate
    from burn_lm_amd.sampling.sampler import Sampler
    cfg, _ = TINIES["B"]
    plain = P.load_model_folder(folders["B"])
    lens = [41, 3, 77, 20, 1, 58, 9]
    prompts = [random_tokens(900 + i, cfg["vocab_size"], n) for i, n in enumerate(lens)]
    want = [P.greedy_generate(plain, p, 6) for p in prompts]
    eng = load(folders["B"], "float32", max_tokens=2048, max_seqs=4)
    steps = []
    real = eng.step
    eng.step = lambda entries: (steps.append([len(t) for _, t, _ in entries]), real(entries))[1]
    whole, whole_stats = generate(eng, prompts, Sampler(temperature=0.0), 6, batch_size=4)
    n_whole = len(steps)
    cut, stats = generate(eng, prompts, Sampler(temperature=0.0), 6, batch_size=4, prompt_budget=32)
    assert [r.tokens for r in cut] == [r.tokens for r in whole] == want
    prompt_steps = [s for s in steps[n_whole:] if max(s) > 1 or sum(s) > len(s)]
    assert all(sum(s) <= 32 for s in prompt_steps) and len(prompt_steps) == -(-sum(lens[:4]) // 32) + -(-sum(lens[4:]) // 32)
    assert stats.prompt_tokens == whole_stats.prompt_tokens == sum(lens)
    assert eng.cache.pages_in_use() == 0


@pytest.mark.parametrize("name,vocab", [("llama3.2-1b", 20008), ("llama3.2-3b", 20008), ("llama3.1-8b", 20008)])
def test_decode_steps_of_100_and_200_sequences_at_the_benchmark_widths(tmp_path, monkeypatch, name, vocab):
    """One layer of each benchmark shape, a batch of 100 and one of 200 short prompts, then six tokens one by one with
    every row's logits wanted, against the plain implementation in both dtypes.  These are the decode steps of 65
    to 256 rows: the fused q/k/v projection with a block for every 64 rows, the output projection on the row-ring
    product at the 1B width, the head of many rows on the matrix-core kernel with a float32 output, and the decode
    attention uncut; the counters say that these kernels were the ones that ran."""
    from burn_lm_amd.config.presets import preset
    from burn_lm_amd.csrc import ops
    cfg = dict(preset(name))
    cfg["num_hidden_layers"] = 1
    cfg["vocab_size"] = vocab
    cfg.pop("eos_token_id", None), cfg.pop("bos_token_id", None)
    folder = make_folder(tmp_path / "shape", cfg, seed=4, std=0.02)
    plain = P.load_model_folder(folder)
    n_dec = 6
    reqs = [random_tokens(70 + i, vocab, 1 + (7 * i) % 23 + n_dec) for i in range(200)]

    def plain_rows(toks, rows):
        h = plain["tok_embeddings"][np.asarray([toks])]
        for lw in plain["layers"]:
            h = P.block(h, lw, plain["cfg"], plain["freqs"], 0)
        return P.rms_norm(h, plain["norm"], plain["cfg"]["eps"])[0][rows] @ plain["output"].T

    want = [plain_rows(r, list(range(len(r) - n_dec, len(r)))) for r in reqs]
    calls = {"qkv": [], "rows": [], "head": [], "attn": []}
    real_qkv, real_rows, real_mfma, real_attn = ops.gemm_rows_qkv_rope, ops.gemm_rows, ops.gemm_mfma, ops.attn_decode
    monkeypatch.setattr(ops, "gemm_rows_qkv_rope", lambda x, *a, **k: (calls["qkv"].append(x.shape[0]), real_qkv(x, *a, **k))[1])
    monkeypatch.setattr(ops, "gemm_rows", lambda a, w, out, **k: (calls["rows"].append(tuple(out.shape)), real_rows(a, w, out, **k))[1])
    monkeypatch.setattr(ops, "gemm_mfma", lambda a, w, out, **k: (calls["head"].append(tuple(out.shape)) if out.dtype == torch.float32
                                                                  and out.dim() == 2 else None, real_mfma(a, w, out, **k))[1])
    monkeypatch.setattr(ops, "attn_decode", lambda q, *a, **k: (calls["attn"].append(q.shape[0]), real_attn(q, *a, **k))[1])
    width = cfg["hidden_size"]
    for dtype, tol in (("float32", 1e-5), ("bfloat16", TOL["bfloat16"])):
        eng = load(folder, dtype, max_tokens=200 * 64, max_seqs=200, graphs=False)
        for n in (100, 200):
            group = list(range(n))
            slots = [eng.open() for _ in group]
            eng.step([(slots[i], reqs[i][:-n_dec], []) for i in group])
            for k in calls:
                del calls[k][:]
            for s in range(n_dec):
                got = eng.step([(slots[i], [reqs[i][len(reqs[i]) - n_dec + s]], [0]) for i in group]).double().cpu().numpy()
                for i in group:
                    assert rel_err(got[i], want[i][s]) <= tol, f"{dtype} batch of {n}: request {i}, decode step {s}"
            if dtype == "bfloat16":
                assert calls["qkv"] == [n] * n_dec, (n, calls["qkv"])
                assert calls["attn"] == [n] * n_dec
                assert calls["head"] == [(n, vocab)] * n_dec, calls["head"]
                ring_o = [s for s in calls["rows"] if s[-1] == width and s[-2] == n]
                assert (len(ring_o) == n_dec) == (width <= 2048), (n, calls["rows"])
            for s in slots:
                eng.close(s)
        del eng
        torch.cuda.empty_cache()


def test_packed_copies_of_the_weights_are_made_when_a_small_step_first_needs_them(folders):
    """A bound bfloat16 matrix is held once until a product of few rows asks for its packed copy: after a prompt of
    many rows none has one, after the first decode step those that such a step multiplies have, and the logits are
    the same with the copies dropped and made again."""
    cfg, _ = TINIES["C"]
    eng = load(folders["C"], "bfloat16", max_tokens=2048, max_seqs=4, graphs=False)
    held = lambda: [w.is_packed for b in eng.model.blocks for w in (b.mixer.w_qkv, b.mixer.w_o, b.feed_forward.w_gate_up,
                                                                     b.feed_forward.w_down)]
    assert all(w.packable for b in eng.model.blocks for w in (b.mixer.w_qkv, b.feed_forward.w_gate_up))
    toks = random_tokens(5, cfg["vocab_size"], 300)
    s = eng.open()
    eng.step([(s, toks[:290], [])])
    assert not any(held()), "a prompt of 290 rows needs no packed copy"
    first = eng.step([(s, [toks[290]], [0])]).clone()
    assert all(held()), "a decode step of one row multiplies every matrix through its packed copy"
    for b in eng.model.blocks:
        for w in (b.mixer.w_qkv, b.mixer.w_o, b.feed_forward.w_gate_up, b.feed_forward.w_down):
            w.drop_packed()
    assert not any(held())
    eng.close(s)
    s = eng.open()
    eng.step([(s, toks[:290], [])])
    again = eng.step([(s, [toks[290]], [0])])
    assert torch.equal(first, again) and all(held())
