"""Long contexts on a one-layer model: with one layer the logits of a row need the keys and values
of every earlier token but the attention of that row only, so the plain formulas can be evaluated
for a few chosen rows of a context of tens of thousands of tokens.  The prompt is fed in pieces of
16,384 tokens; the chosen rows lie at the llama3 scaling's original context length (8,191 and
8,192), inside a later piece, at the prompt's end, and in the decode steps that follow, which run
as a batch of two sequences of very unequal lengths (cut decode attention, hundreds of pages)."""
import numpy as np
import pytest

import plain_llama as P
from helpers import TOL, make_folder, random_tokens, rel_err

pytestmark = pytest.mark.gpu


def plain_rows(m, toks, rows):
    """Logits of the given rows of a one-layer model, each part by its plain function."""
    cfg = m["cfg"]
    nh, nkv, hd = cfg["n_heads"], cfg["n_kv_heads"], cfg["head_dim"]
    lw = m["layers"][0]
    h = m["tok_embeddings"][np.asarray(toks)]
    x = P.rms_norm(h, lw["attention_norm"], cfg["eps"])
    T = len(toks)
    k = P.rope_interleaved((x @ lw["wk"].T).reshape(T, nkv, hd).swapaxes(0, 1), np.arange(T), m["freqs"])
    v = (x @ lw["wv"].T).reshape(T, nkv, hd).swapaxes(0, 1)
    out = []
    for r in rows:
        q = P.rope_interleaved((x[r] @ lw["wq"].T).reshape(1, nh, 1, hd), np.array([r]), m["freqs"])
        o = P.scaled_attention(q, k[None, :, :r + 1], v[None, :, :r + 1], None).reshape(nh * hd)
        hr = h[r] + o @ lw["wo"].T
        hr = hr + P.swiglu_feed_forward(P.rms_norm(hr, lw["ffn_norm"], cfg["eps"]), lw["w1"], lw["w3"], lw["w2"])
        out.append(P.rms_norm(hr, m["norm"], cfg["eps"]) @ m["output"].T)
    return np.stack(out)


@pytest.mark.parametrize("hd,nh,nkv,T", [(64, 8, 2, 40000), (128, 4, 1, 70000)])
def test_long_contexts(tmp_path, hd, nh, nkv, T):
    from burn_lm_amd.engine.loading import load_engine
    cfg = dict(architectures=["LlamaForCausalLM"], hidden_size=512, intermediate_size=1024, num_hidden_layers=1,
               num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd, vocab_size=1000,
               max_position_embeddings=131072, rms_norm_eps=1e-5, rope_theta=500000.0, tie_word_embeddings=True,
               rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                 original_max_position_embeddings=8192))
    folder = make_folder(tmp_path / "m", cfg, seed=hd, std=0.06)
    m = P.load_model_folder(folder)
    toks = random_tokens(7 + hd, 1000, T + 6)
    inside = (8191, 8192, 20000)
    decoded = (T, T + 1, T + 5)
    want = plain_rows(m, toks, list(inside) + [T - 1] + list(decoded))
    for dtype, tol in (("float32", 1e-5), ("bfloat16", TOL["bfloat16"])):
        eng = load_engine(folder, dtype=dtype, max_tokens=T + 2048, max_seqs=2)
        s, other = eng.open(), eng.open()
        fed, got = 0, {}
        while fed < T:
            n = min(16384, T - fed)
            rows = [r - fed for r in inside if fed <= r < fed + n] + ([n - 1] if fed + n == T else [])
            out = eng.step([(s, toks[fed:fed + n], rows)])
            for j, r in enumerate(rows):
                got[fed + r] = out[j].double().cpu().numpy()
            fed += n
        eng.step([(other, toks[:70], [69])])
        for j in range(6):
            out = eng.step([(other, [toks[70 + j]], [0]), (s, [toks[T + j]], [0])])
            got[T + j] = out[1].double().cpu().numpy()
        for j, r in enumerate(list(inside) + [T - 1] + list(decoded)):
            assert rel_err(got[r], want[j]) <= tol, f"{dtype}: row {r} of a context of {T}"
        del eng
