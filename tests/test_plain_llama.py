"""Pins the plain implementation by what fixes it beside the reference's text: the vectors
its own tests hold, special cases that reduce to a library routine, and invariants.  Each is
chosen so that a plausible mistake (wrong sign or pairing, eps outside the root, a norm in the
wrong place, scale before the product) fails it."""
import math

import numpy as np
import torch

import plain_llama as P


def range_init(shape_in_out):
    """Reference fixture ``Reinitializer::range_float(0, 5)``: arange(n) * 5/n in the
    tensor's own ``[d_in, d_out]`` element order (crates/burn-lm-llama/src/lib.rs:142-148,
    199-205).  Returned as the ``[d_out, d_in]`` matrix the plain functions take."""
    n = int(np.prod(shape_in_out))
    w = (np.arange(n, dtype=np.float64) * (5.0 / n)).reshape(shape_in_out)
    return w.T if w.ndim == 2 else w


# ---- vectors held by the reference's own tests -----------------------------------------
def test_rms_norm_vector():
    # crates/burn-lm-llama/src/nn/transformer.rs:278-297 (eps 1e-5, gamma 1, rel 5 %)
    x = np.array([[0.0025997162, 0.0030002594, -0.006000519, 0.006000519],
                  [0.0010004044, 0.00080013275, 0.0015001297, -0.01600647]])
    want = np.array([[0.45996094, 0.5307617, -1.0615234, 1.0615234],
                     [0.11553955, 0.09240723, 0.17321777, -1.8486328]])
    got = P.rms_norm(x, np.ones(4), 1e-5)
    np.testing.assert_allclose(got, want, rtol=5e-3)
    # inputs are ~1e-3, so eps matters: eps outside the root or missing must fail
    wrong = x / (np.sqrt(np.mean(x * x, -1, keepdims=True)) + 1e-5)
    assert np.max(np.abs(wrong / want - 1)) > 0.05


def test_rope_vector():
    # crates/burn-lm-llama/src/nn/pos_encoding.rs:151-179: head_dim 2, theta 5e5, scaling 32
    freqs = P.llama3_frequency_scaling(P.rope_base_frequencies(2, 500000.0), scale_factor=32.0)
    x = np.array([[[[-0.60253906, -0.035308838], [0.41357422, 0.15100098]],
                   [[-0.044677734, -0.094177246], [0.60546875, 0.2442627]]]])
    want = np.array([[[[-0.60253906, -0.035308838], [0.09643555, 0.42944336]],
                      [[-0.044677734, -0.094177246], [0.12194824, 0.64160156]]]])
    got = P.rope_interleaved(x, [0, 1], freqs)
    np.testing.assert_allclose(got, want, rtol=5e-3)  # vector carries half-precision error
    # the opposite rotation sense must fail
    bad = P.rope_interleaved(x, [0, -1], freqs)
    assert np.max(np.abs(bad - want)) > 0.1


def test_feed_forward_vector():
    # crates/burn-lm-llama/src/nn/fftn.rs:57-92
    x = np.arange(16, dtype=np.float64).reshape(2, 2, 4)
    want = np.array([[[8661.133, 9206.727, 9752.319, 10297.912],
                      [73848.63, 78356.14, 82863.65, 87371.16]],
                     [[202911.13, 215216.48, 227521.86, 239827.2],
                      [395848.63, 419787.78, 443726.94, 467666.06]]])
    got = P.swiglu_feed_forward(x, range_init((4, 8)), range_init((4, 8)), range_init((8, 4)))
    np.testing.assert_allclose(got, want, rtol=1e-6)


def _reference_test_model():
    # crates/burn-lm-llama/src/nn/transformer.rs:299-349: TransformerConfig::new(8,2,8,16,2,1)
    layers = [dict(wq=range_init((8, 8)), wk=range_init((8, 4)), wv=range_init((8, 4)),
                   wo=range_init((8, 8)), w1=range_init((8, 16)), w3=range_init((8, 16)),
                   w2=range_init((16, 8)), attention_norm=range_init((8,)),
                   ffn_norm=range_init((8,))) for _ in range(2)]
    return dict(cfg=dict(n_heads=2, n_kv_heads=1, head_dim=4, eps=1e-5),
                freqs=P.rope_base_frequencies(4, 10000.0),
                tok_embeddings=(np.arange(64) * 5.0 / 64).reshape(8, 8),
                layers=layers, norm=range_init((8,)), output=range_init((8, 8)), vocab=8)


def test_whole_model_vector():
    want = np.array([[[56.37573, 57.77283, 59.169933, 60.567043, 61.964146, 63.361248, 64.758354, 66.15546],
                      [56.374626, 57.77171, 59.168793, 60.56588, 61.962963, 63.360046, 64.75713, 66.15422]],
                     [[56.374252, 57.771328, 59.168407, 60.565487, 61.962566, 63.359642, 64.75672, 66.1538],
                      [56.37408, 57.771156, 59.168232, 60.565304, 61.96238, 63.359455, 64.75653, 66.15361]]])
    got = P.transformer_forward([[0, 1], [2, 3]], _reference_test_model())
    np.testing.assert_allclose(got, want, rtol=2e-6)


def test_temperature_vector():
    # crates/burn-lm-llama/src/generation/generate.rs:121-137 (values carry half-precision error)
    got = P.temperature_softmax([[21.3125, 19.859375, 19.0625, 18.75, 18.171875]], 0.6)
    want = [[0.8691406, 0.07836914, 0.020767212, 0.0124053955, 0.0047035217]]
    np.testing.assert_allclose(got, want, rtol=0.05)
    assert abs(got.sum() - 1) < 1e-12


# ---- special cases that reduce to a library routine ------------------------------------
def test_attention_equals_library_sdpa():
    rng = np.random.default_rng(0)
    b, nh, nkv, t, hd = 2, 6, 2, 7, 8
    q = rng.standard_normal((b, nh, t, hd))
    k = rng.standard_normal((b, nkv, t, hd))
    v = rng.standard_normal((b, nkv, t, hd))
    got = P.scaled_attention(q, k, v, P.hidden_mask(t, t))
    tq, tk, tv = (torch.from_numpy(a) for a in (q, k, v))
    rep = nh // nkv
    want = torch.nn.functional.scaled_dot_product_attention(
        tq, tk.repeat_interleave(rep, 1), tv.repeat_interleave(rep, 1), is_causal=True)
    np.testing.assert_allclose(got, want.numpy(), rtol=1e-10, atol=1e-12)
    # grouping by h % nkv instead of h // rep must differ
    wrong = torch.nn.functional.scaled_dot_product_attention(
        tq, tk.repeat(1, rep, 1, 1), tv.repeat(1, rep, 1, 1), is_causal=True)
    assert np.max(np.abs(got - wrong.numpy())) > 1e-2


def test_attention_layer_without_rotation_is_library_attention():
    # zero frequencies = no rotation; one head; equals SDPA on the projections
    rng = np.random.default_rng(1)
    d, t = 8, 5
    x = rng.standard_normal((1, t, d))
    wq, wk, wv, wo = (rng.standard_normal((d, d)) for _ in range(4))
    got = P.attention_layer(x, wq, wk, wv, wo, 1, 1, d, np.zeros(d // 2))
    tx = torch.from_numpy(x)
    o = torch.nn.functional.scaled_dot_product_attention(
        (tx @ torch.from_numpy(wq).T)[:, None], (tx @ torch.from_numpy(wk).T)[:, None],
        (tx @ torch.from_numpy(wv).T)[:, None], is_causal=True)[:, 0]
    np.testing.assert_allclose(got, (o @ torch.from_numpy(wo).T).numpy(), rtol=1e-10)


def test_rope_is_complex_multiplication():
    rng = np.random.default_rng(2)
    hd, t = 12, 9
    x = rng.standard_normal((3, t, hd))
    freqs = P.rope_base_frequencies(hd, 500000.0)
    pos = np.arange(5, 5 + t)
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * pos[:, None] * freqs[None, :])
    got = P.rope_interleaved(x, pos, freqs)
    np.testing.assert_allclose(got[..., 0::2], z.real, atol=1e-12)
    np.testing.assert_allclose(got[..., 1::2], z.imag, atol=1e-12)


def test_silu_matches_library():
    z = np.linspace(-6, 6, 25)
    np.testing.assert_allclose(P.silu(z), torch.nn.functional.silu(torch.from_numpy(z)).numpy(),
                               rtol=1e-12)


# ---- invariants --------------------------------------------------------------------------
def test_rope_scores_depend_on_distance_only():
    rng = np.random.default_rng(3)
    hd = 16
    freqs = P.llama3_frequency_scaling(P.rope_base_frequencies(hd, 500000.0), 8, 1, 4, 32)
    q, k = rng.standard_normal((1, hd)), rng.standard_normal((1, hd))
    base = P.rope_interleaved(q, [7], freqs) @ P.rope_interleaved(k, [3], freqs).T
    moved = P.rope_interleaved(q, [107], freqs) @ P.rope_interleaved(k, [103], freqs).T
    np.testing.assert_allclose(base, moved, rtol=1e-9)
    other = P.rope_interleaved(q, [107], freqs) @ P.rope_interleaved(k, [102], freqs).T
    assert abs(float(base) - float(other)) > 1e-3


def test_shift_of_all_positions_changes_no_logit():
    model = _random_model(seed=5)
    ids = [[3, 1, 4, 1, 5, 9, 2, 6]]
    a = P.transformer_forward(ids, model, start_pos=0)
    b = P.transformer_forward(ids, model, start_pos=37)
    np.testing.assert_allclose(a, b, rtol=1e-8, atol=1e-10)


def test_llama3_scaling_branches_and_continuity():
    # head_dim 24, theta 5e5, (8, 1, 4, 32): lane 0 kept, lane 1 blended, lanes 2.. divided
    base = P.rope_base_frequencies(24, 500000.0)
    sc = P.llama3_frequency_scaling(base, 8, 1, 4, 32)
    assert sc[0] == base[0]
    assert base[1] / 8 < sc[1] < base[1]
    np.testing.assert_allclose(sc[2:], base[2:] / 8, rtol=1e-12)
    # factor 1 is the identity
    np.testing.assert_allclose(P.llama3_frequency_scaling(base, 1, 1, 4, 32), base, rtol=1e-12)
    # continuous at both band edges: wavelen = old/high -> unchanged, wavelen = old/low -> /factor
    hi = np.array([2 * math.pi / (32 / 4)])
    lo = np.array([2 * math.pi / (32 / 1)])
    np.testing.assert_allclose(P.llama3_frequency_scaling(hi, 8, 1, 4, 32), hi, rtol=1e-9)
    np.testing.assert_allclose(P.llama3_frequency_scaling(lo, 8, 1, 4, 32), lo / 8, rtol=1e-9)
    # defaults of the reference (pos_encoding.rs:93-100)
    np.testing.assert_allclose(P.llama3_frequency_scaling(base), P.llama3_frequency_scaling(base, 8, 1, 4, 8192))


def test_interleaved_on_permuted_rows_equals_half_split_on_raw_rows():
    # the reason for import.rs:94-127: HF stores (first half, second half) pairs
    rng = np.random.default_rng(4)
    nh, hd, d, t = 3, 8, 10, 6
    w = rng.standard_normal((nh * hd, d))
    x = rng.standard_normal((t, d))
    freqs = P.rope_base_frequencies(hd, 10000.0)
    pos = np.arange(t)
    a = P.rope_interleaved((x @ P.permute_hf_rows(w, nh).T).reshape(t, nh, hd).swapaxes(0, 1), pos, freqs)
    raw = (x @ w.T).reshape(t, nh, hd).swapaxes(0, 1)
    ang = pos[:, None] * freqs[None, :]
    x0, x1 = raw[..., : hd // 2], raw[..., hd // 2:]
    b0 = x0 * np.cos(ang) - x1 * np.sin(ang)
    b1 = x0 * np.sin(ang) + x1 * np.cos(ang)
    # scores between heads are what matters; compare lane-by-lane after un-permuting
    np.testing.assert_allclose(a[..., 0::2], b0, atol=1e-12)
    np.testing.assert_allclose(a[..., 1::2], b1, atol=1e-12)


def test_future_tokens_never_change_earlier_logits():
    model = _random_model(seed=6)
    a = P.transformer_forward([[5, 4, 3, 2, 1, 0]], model)
    b = P.transformer_forward([[5, 4, 3, 7, 7, 7]], model)
    np.testing.assert_allclose(a[0, :3], b[0, :3], rtol=1e-10)
    assert np.max(np.abs(a[0, 3:] - b[0, 3:])) > 1e-6


def test_single_token_attention_returns_value():
    q = np.ones((1, 2, 1, 4)); k = np.full((1, 1, 1, 4), 3.0); v = np.arange(4.0).reshape(1, 1, 1, 4)
    np.testing.assert_allclose(P.scaled_attention(q, k, v, P.hidden_mask(1, 1))[0, :, 0], [[0, 1, 2, 3]] * 2)


def test_zero_query_gives_mean_of_visible_values():
    rng = np.random.default_rng(7)
    t, hd = 5, 4
    k, v = rng.standard_normal((1, 1, t, hd)), rng.standard_normal((1, 1, t, hd))
    o = P.scaled_attention(np.zeros((1, 1, t, hd)), k, v, P.hidden_mask(t, t))
    for i in range(t):
        np.testing.assert_allclose(o[0, 0, i], v[0, 0, : i + 1].mean(0), rtol=1e-12)


def test_hidden_mask_matches_reference_rule():
    # tril_mask([T, S], offset S-T): hidden where j > i + S - T (transformer.rs:168-180)
    m = P.hidden_mask(3, 5)
    assert m.tolist() == [[False, False, False, True, True],
                          [False, False, False, False, True],
                          [False, False, False, False, False]]
    assert P.hidden_mask(1, 9) is None


def test_norm_placement_is_pre_norm():
    # with zero attention and ffn output weights the block is the identity: a post-norm would not be
    model = _random_model(seed=8)
    lw = dict(model["layers"][0])
    lw["wo"] = np.zeros_like(lw["wo"]); lw["w2"] = np.zeros_like(lw["w2"])
    x = np.random.default_rng(9).standard_normal((1, 4, model["tok_embeddings"].shape[1]))
    np.testing.assert_allclose(P.block(x, lw, model["cfg"], model["freqs"]), x)


def test_top_p_keeps_the_token_that_crosses_p():
    # generation/sampling.rs:56-63: a token is kept while the mass before it is < p
    probs = np.array([0.1, 0.5, 0.15, 0.25])
    assert P.top_p_keep(probs, 0.7) == [1, 3]
    assert P.top_p_keep(probs, 0.75) == [1, 3]
    assert P.top_p_keep(probs, 0.76) == [1, 3, 2]
    assert P.top_p_keep(probs, 1.0) == [1, 3, 2, 0]


def test_greedy_stops_on_stop_token():
    model = _random_model(seed=10)
    free = P.greedy_generate(model, [1, 2, 3], 6)
    assert len(free) == 6
    stopped = P.greedy_generate(model, [1, 2, 3], 6, stop_ids=(free[2],))
    assert stopped == free[: free.index(free[2]) + 1]


def _random_model(seed, d=16, nh=4, nkv=2, hd=4, inter=24, vocab=11, n_layers=2):
    rng = np.random.default_rng(seed)
    g = lambda *s: rng.standard_normal(s) * 0.3
    layers = [dict(wq=g(nh * hd, d), wk=g(nkv * hd, d), wv=g(nkv * hd, d), wo=g(d, nh * hd),
                   w1=g(inter, d), w3=g(inter, d), w2=g(d, inter),
                   attention_norm=1 + g(d), ffn_norm=1 + g(d)) for _ in range(n_layers)]
    return dict(cfg=dict(n_heads=nh, n_kv_heads=nkv, head_dim=hd, eps=1e-5),
                freqs=P.rope_base_frequencies(hd, 10000.0), tok_embeddings=g(vocab, d),
                layers=layers, norm=1 + g(d), output=g(vocab, d), vocab=vocab)
