"""Configurations drawn at random: every size anew for each seed (head sizes in steps of 16 up to 256,
any number of heads and groups, widths that are no multiple of the head count times the head size or
of 8, odd inner widths and vocabularies, one to three layers, eps, theta and frequency scaling), each
run through a random schedule of steps (prompts whole and in pieces, tokens one by one, up to 40
sequences at once, any rows wanted) in 32-bit and in bfloat16 against the plain implementation.

The two fixed tiny configurations pin the paths that the other tests name; this one is for the sizes
nobody thought of: a kernel either takes a size, refuses it with an error at load, or this fails."""
import numpy as np
import pytest

import plain_llama as P
from helpers import TOL, make_folder, random_tokens, rel_err

pytestmark = pytest.mark.gpu


def draw_config(rng):
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 256]))
    nkv = int(rng.choice([1, 2, 3, 4, 8]))
    nh = nkv * int(rng.choice([1, 1, 2, 3, 4, 5, 8]))
    while nh * hd > 2048:       # halve both counts, keep the heads a multiple of the groups
        nkv = max(1, nkv // 2)
        nh = max(nkv, nh // 2 // nkv * nkv)
    cfg = dict(architectures=["LlamaForCausalLM"], num_attention_heads=nh, num_key_value_heads=nkv,
               num_hidden_layers=int(rng.integers(1, 4)), vocab_size=int(rng.integers(50, 20000)),
               max_position_embeddings=int(rng.choice([512, 1024, 4096])),
               rms_norm_eps=float(rng.choice([1e-5, 1e-6, 1e-3])), rope_theta=float(rng.choice([1e4, 5e5, 1e6])),
               tie_word_embeddings=bool(rng.random() < 0.5))
    if rng.random() < 0.5:
        cfg["hidden_size"] = nh * hd
    else:                       # a width of its own, the head size given beside it
        step = int(rng.choice([2, 8, 8, 16, 64]))
        cfg["hidden_size"] = int(rng.integers(64 // step, 1024 // step + 1)) * step
        cfg["head_dim"] = hd
    step = int(rng.choice([1, 2, 8, 8, 32]))
    cfg["intermediate_size"] = int(rng.integers(32 // step + 1, 2000 // step + 1)) * step
    if rng.random() < 0.5:
        cfg["rope_scaling"] = dict(rope_type="llama3", factor=float(rng.choice([2.0, 8.0, 32.0])),
                                   low_freq_factor=float(rng.choice([1.0, 2.0])), high_freq_factor=float(rng.choice([4.0, 8.0])),
                                   original_max_position_embeddings=int(rng.choice([64, 256, 8192])))
    return cfg


def run_schedule(eng, plain, vocab, rng, max_seqs, last_only, dtype, iterations=14):
    """Random steps on up to max_seqs sequences; every wanted row against the plain implementation.
    Returns the number of rows compared."""
    from burn_lm_amd.cache.cache import CacheFull
    live, compared = {}, 0        # slot -> [tokens, tokens fed, the plain implementation's logits]
    for _ in range(iterations):
        while len(live) < max_seqs and (not live or rng.random() < 0.7):
            try:
                s = eng.open()
            except CacheFull:
                break
            live[s] = [random_tokens(int(rng.integers(1 << 30)), vocab, int(rng.integers(1, 200))), 0, None]
        picks = [s for s in live if rng.random() < 0.85]
        rng.shuffle(picks)
        one_each = rng.random() < 0.5      # a decode step: one token for every sequence that has begun
        entries, expect = [], []
        for s in picks:
            toks, fed, _ = live[s]
            if fed == len(toks):
                continue
            n = 1 if (one_each and fed > 0) else int(min(len(toks) - fed, rng.choice([1, 2, 17, 64, 65, 130])))
            rows = [n - 1] if last_only else sorted({int(r) for r in rng.integers(0, n, size=int(rng.integers(0, 3)))})
            entries.append((s, toks[fed:fed + n], rows))
            expect += [(s, fed + r) for r in rows]
        if not entries:
            continue
        try:
            got = eng.step(entries)
        except CacheFull:
            victim = max(live, key=lambda s: live[s][1])
            eng.close(victim)
            del live[victim]
            continue
        for s, t, _ in entries:
            live[s][1] += len(t)
        if got is not None:
            got = got.double().cpu().numpy()
            assert got.shape[0] == len(expect)
            for row, (s, pos) in zip(got, expect):
                if live[s][2] is None:
                    live[s][2] = P.transformer_forward([live[s][0]], plain)[0]
                err = rel_err(row, live[s][2][pos])
                assert err <= TOL[dtype], (dtype, err, pos, len(live[s][0]), [(len(t), w) for _, t, w in entries])
                compared += 1
        for s in list(live):
            if live[s][1] == len(live[s][0]) or rng.random() < 0.05:
                eng.close(s)
                del live[s]
    for s in list(live):
        eng.close(s)
    assert eng.cache.pages_in_use() == 0
    return compared


@pytest.mark.parametrize("seed", range(24))
def test_a_drawn_configuration_through_a_random_schedule(seed, tmp_path):
    from burn_lm_amd.engine.loading import load_engine
    rng = np.random.default_rng(9000 + seed)
    cfg = draw_config(rng)
    print(cfg)
    # weights scaled so that a layer's products keep the activations' size, as a trained model's do: at
    # 0.05 a width of 1,500 makes the attention so sharp that exact arithmetic between bfloat16
    # roundings (the plain implementation with roundings, on the CPU) is 0.03-0.07 of the largest logit
    # from the exact result, beyond the tolerance, with no engine involved
    folder = make_folder(tmp_path / "m", cfg, seed, std=min(0.05, 0.9 / cfg["hidden_size"] ** 0.5))
    plain = P.load_model_folder(folder)
    compared = 0
    for dtype in ("bfloat16", "float32"):
        max_seqs = int(rng.choice([3, 12, 40]))
        eng = load_engine(folder, dtype=dtype, max_tokens=int(rng.choice([2048, 4096])), max_seqs=max_seqs,
                          max_context=min(cfg["max_position_embeddings"], 512))
        compared += run_schedule(eng, plain, cfg["vocab_size"], rng, max_seqs, last_only=seed % 2 == 0, dtype=dtype)
        del eng
    assert compared > 0
