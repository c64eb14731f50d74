"""Each part alone, built by its registered kind with weights of its own, against the plain
function of the same part; and a block put together from them."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P

PAGE = 64

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2}


@pytest.fixture(scope="module", params=[torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def rt(request):
    from burn_lm_amd.engine.runtime import Runtime
    import burn_lm_amd  # noqa: F401
    return Runtime(dtype=request.param, device="cuda:0")


def rel(got, want):
    got = got.double().cpu().numpy()
    return float(np.abs(got - want).max() / np.abs(want).max())


def weights(rt, seed, **shapes):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in shapes.items():
        t = torch.randn(shape, generator=g) * (0.3 if len(shape) == 2 else 0.2)
        if len(shape) == 1:
            t = t + 1
        out[name] = t.to(rt.dtype)
    return out, {k: v.double().numpy() for k, v in out.items()}


def on_gpu(t):
    return {k: v.to("cuda") for k, v in t.items()}


def test_rmsnorm_part(rt):
    from burn_lm_amd import registry
    t, tn = weights(rt, 0, w=(150,))
    norm = registry.part("norm", "rmsnorm")(dict(width=150, eps=1e-4), dict(weight="w"))
    assert norm.tensor_specs()["w"].shape == (150,)
    norm.bind(on_gpu(t), rt)
    g = torch.Generator().manual_seed(1)
    h = torch.randn(9, 150, generator=g) * 0.05
    d = (torch.randn(9, 150, generator=g) * 0.05).to(rt.dtype)
    hd = h.to("cuda")
    x = norm.add_norm(hd, d.to("cuda"))
    want = P.rms_norm((h + d.float()).double().numpy(), tn["w"], 1e-4)
    assert rel(x, want) <= TOL[rt.dtype] and x.dtype == rt.dtype
    assert torch.equal(hd.cpu(), h + d.float())


def test_rotary_part_table_follows_the_reference_scaling(rt):
    from burn_lm_amd import registry
    rope = registry.part("position", "rope")(dict(head_dim=24, theta=500000.0, pairing="interleaved",
                                                  scaling=(8.0, 1.0, 4.0, 32)), {})
    rope.bind({}, rt)
    rope.prepare(300, rt)
    f = P.llama3_frequency_scaling(P.rope_base_frequencies(24, 500000.0), 8.0, 1.0, 4.0, 32)
    np.testing.assert_allclose(rope.freqs, f, rtol=1e-12)
    ang = np.arange(300)[:, None] * f[None, :]
    tab = rope.table.cpu().double().numpy()
    np.testing.assert_allclose(tab[..., 0], np.cos(ang), atol=1e-7)
    np.testing.assert_allclose(tab[..., 1], np.sin(ang), atol=1e-7)
    plain = registry.part("position", "rope")(dict(head_dim=24, theta=500000.0, pairing="half", scaling=None), {})
    plain.bind({}, rt)
    np.testing.assert_allclose(plain.freqs, P.rope_base_frequencies(24, 500000.0), rtol=1e-12)
    with pytest.raises(ValueError, match="pairing"):
        registry.part("position", "rope")(dict(head_dim=8, theta=1e4, pairing="odd"), {}).bind({}, rt)


@pytest.mark.parametrize("pairing", ["interleaved", "half"])
@pytest.mark.parametrize("heads,kv_heads,hd", [(4, 2, 16), (6, 1, 24), (3, 3, 40)])
def test_attention_part(rt, pairing, heads, kv_heads, hd):
    """Whole sequences in one step, then the same sequences cut in two steps, against the plain
    attention sub-layer.  With pairing "half" the weights are in the Hugging Face row order and the
    plain side permutes them as the reference does on import."""
    from burn_lm_amd import registry
    from burn_lm_amd.cache.cache import Cache
    from burn_lm_amd.engine.batch import build_step
    D = 72
    t, tn = weights(rt, 2, q=(heads * hd, D), k=(kv_heads * hd, D), v=(kv_heads * hd, D), o=(D, heads * hd))
    rope = registry.part("position", "rope")(dict(head_dim=hd, theta=10000.0, pairing=pairing, scaling=None), {})
    rope.bind({}, rt)
    rope.prepare(256, rt)
    attn = registry.part("mixer", "attention")(
        dict(width=D, heads=heads, kv_heads=kv_heads, head_dim=hd, scale=1 / math.sqrt(hd), window=0, position=rope),
        dict(q="q", k="k", v="v", o="o"))
    assert attn.tensor_specs()["k"].shape == (kv_heads * hd, D)
    attn.bind(on_gpu(t), rt)
    wq, wk = tn["q"], tn["k"]
    if pairing == "half":
        wq, wk = P.permute_hf_rows(wq, heads), P.permute_hf_rows(wk, kv_heads)
    freqs = P.rope_base_frequencies(hd, 10000.0)
    g = torch.Generator().manual_seed(3)
    lens = [37, 1, 20]
    xs = [(torch.randn(n, D, generator=g)).to(rt.dtype) for n in lens]
    want = [P.attention_layer(x.double().numpy()[None], wq, wk, tn["v"], tn["o"], heads, kv_heads, hd, freqs)[0]
            for x in xs]
    for cuts in ([37, 1, 20], [30, 1, 7]):
        cache = Cache([attn.cache_need()], [None], 1024, 8, 256, PAGE, rt.dtype, rt.device)
        slots = [cache.open() for _ in lens]
        done = [0, 0, 0]
        outs = [[], [], []]
        while any(d < n for d, n in zip(done, lens)):
            entries, idx = [], []
            for i, (d, n) in enumerate(zip(done, lens)):
                if d < n:
                    c = cuts[i] if d == 0 else n - d
                    entries.append((slots[i], [0] * c, []))
                    idx.append((i, d, c))
            cache.reserve([(s, len(tk)) for s, tk, _ in entries])
            step = build_step(entries, cache, rt.device)
            x = torch.cat([xs[i][d:d + c] for i, d, c in idx]).to("cuda")
            y = attn.forward(x, step, cache.views[0])
            o = 0
            for i, d, c in idx:
                outs[i].append(y[o:o + c]); o += c
                cache.advance(slots[i], c); done[i] += c
        for i in range(3):
            assert rel(torch.cat(outs[i]), want[i]) <= TOL[rt.dtype], f"sequence {i}, cuts {cuts}"


@pytest.mark.parametrize("pairing,heads,kv_heads,hd,turning", [("interleaved", 4, 2, 32, 8), ("half", 6, 3, 24, 16),
                                                               ("half", 2, 1, 64, 32), ("interleaved", 3, 1, 48, 46)])
def test_attention_part_with_only_part_of_each_head_rotated(rt, pairing, heads, kv_heads, hd, turning):
    """rotary_dim: the first `turning` lanes of every head turn by theta^(-2i/turning), the rest pass through.  The plain side
    rotates those lanes itself (adjacent pairs, or pairs half the turning lanes apart) and leaves the others alone; a prompt step of
    unequal sequences, then single tokens."""
    from burn_lm_amd import registry
    from burn_lm_amd.cache.cache import Cache
    from burn_lm_amd.engine.batch import build_step
    D = 64
    t, tn = weights(rt, 5, q=(heads * hd, D), k=(kv_heads * hd, D), v=(kv_heads * hd, D), o=(D, heads * hd))
    rope = registry.part("position", "rope")(dict(head_dim=hd, theta=10000.0, pairing=pairing, scaling=None, rotary_dim=turning), {})
    rope.bind({}, rt)
    rope.prepare(256, rt)
    assert rope.freqs.shape == (hd // 2,) and np.all(rope.freqs[turning // 2:] == 0)
    np.testing.assert_allclose(rope.freqs[: turning // 2], P.rope_base_frequencies(turning, 10000.0), rtol=1e-12)
    attn = registry.part("mixer", "attention")(
        dict(width=D, heads=heads, kv_heads=kv_heads, head_dim=hd, scale=1 / math.sqrt(hd), window=0, position=rope),
        dict(q="q", k="k", v="v", o="o"))
    attn.bind(on_gpu(t), rt)
    freqs = P.rope_base_frequencies(turning, 10000.0)

    def turn(x, pos):     # x [heads, T, hd]
        a = pos[:, None] * freqs[None, :]
        c, s = np.cos(a), np.sin(a)
        head, tail = x[..., :turning], x[..., turning:]
        out = np.empty_like(head)
        if pairing == "interleaved":
            e, o = head[..., 0::2], head[..., 1::2]
            out[..., 0::2], out[..., 1::2] = e * c - o * s, e * s + o * c
        else:
            lo, hi = head[..., : turning // 2], head[..., turning // 2:]
            out[..., : turning // 2], out[..., turning // 2:] = lo * c - hi * s, lo * s + hi * c
        return np.concatenate([out, tail], axis=-1)

    def plain(x):
        T = x.shape[0]
        pos = np.arange(T, dtype=np.float64)
        q = (x @ tn["q"].T).reshape(T, heads, hd).swapaxes(0, 1)
        k = (x @ tn["k"].T).reshape(T, kv_heads, hd).swapaxes(0, 1)
        v = (x @ tn["v"].T).reshape(T, kv_heads, hd).swapaxes(0, 1)
        o = P.scaled_attention(turn(q, pos)[None], turn(k, pos)[None], v[None], P.hidden_mask(T, T))[0]
        return o.swapaxes(0, 1).reshape(T, heads * hd) @ tn["o"].T

    g = torch.Generator().manual_seed(8)
    lens = [70, 3, 33]
    xs = [(torch.randn(n, D, generator=g)).to(rt.dtype) for n in lens]
    want = [plain(x.double().numpy()) for x in xs]
    cache = Cache([attn.cache_need()], [None], 1024, 8, 256, PAGE, rt.dtype, rt.device)
    slots = [cache.open() for _ in lens]
    first = [n - 2 for n in lens]
    outs = [[], [], []]
    for chunk in range(3):
        entries = [(s, [0] * (first[i] if chunk == 0 else 1), []) for i, s in enumerate(slots)]
        cache.reserve([(s, len(tk)) for s, tk, _ in entries])
        step = build_step(entries, cache, rt.device)
        at = [0 if chunk == 0 else first[i] + chunk - 1 for i in range(3)]
        x = torch.cat([xs[i][at[i]: at[i] + len(entries[i][1])] for i in range(3)]).to("cuda")
        y = attn.forward(x, step, cache.views[0])
        o = 0
        for i in range(3):
            n = len(entries[i][1])
            outs[i].append(y[o:o + n]); o += n
            cache.advance(slots[i], n)
    for i in range(3):
        assert rel(torch.cat(outs[i]), want[i]) <= TOL[rt.dtype], f"sequence {i}"
    with pytest.raises(ValueError, match="rotary_dim"):
        registry.part("position", "rope")(dict(head_dim=16, theta=1e4, pairing="half", rotary_dim=7), {}).bind({}, rt)
    if pairing == "half":
        with pytest.raises(ValueError, match="for_projection"):
            rope.encode_and_store(None, None, None, heads, kv_heads, hd)


def test_swiglu_part(rt):
    from burn_lm_amd import registry
    t, tn = weights(rt, 4, g=(200, 72), u=(200, 72), d=(72, 200))
    ffn = registry.part("feed_forward", "swiglu")(dict(width=72, inner=200), dict(gate="g", up="u", down="d"))
    ffn.bind(on_gpu(t), rt)
    for rows in (3, 40):   # few rows take the skinny product, many the other one
        x = (torch.randn(rows, 72, generator=torch.Generator().manual_seed(5))).to(rt.dtype)
        want = P.swiglu_feed_forward(x.double().numpy(), tn["g"], tn["u"], tn["d"])
        assert rel(ffn.forward(x.to("cuda"), None), want) <= TOL[rt.dtype]
    # swapping gate and up must show: silu is on the gate
    wrong = P.swiglu_feed_forward(x.double().numpy(), tn["u"], tn["g"], tn["d"])
    assert np.abs(wrong - want).max() / np.abs(want).max() > 0.1
    if rt.dtype == torch.bfloat16:
        # many rows with the gating fused into the matrix-core product (off unless asked for)
        rt.fused_gate_up_rows = (65, 4096)
        try:
            x = (torch.randn(300, 72, generator=torch.Generator().manual_seed(6))).to(rt.dtype)
            want = P.swiglu_feed_forward(x.double().numpy(), tn["g"], tn["u"], tn["d"])
            assert rel(ffn.forward(x.to("cuda"), None), want) <= TOL[rt.dtype]
        finally:
            rt.fused_gate_up_rows = (0, -1)


def test_embedding_and_head_parts(rt):
    from burn_lm_amd import registry
    t, tn = weights(rt, 6, e=(301, 72), h=(301, 72))
    emb = registry.part("embedding", "table")(dict(vocab=301, width=72), dict(weight="e"))
    emb.bind(on_gpu(t), rt)
    ids = torch.tensor([300, 0, 17], dtype=torch.int32, device="cuda")
    h = emb.forward(ids)
    assert h.dtype == torch.float32 and torch.equal(h.cpu(), t["e"][[300, 0, 17]].float())
    head = registry.part("head", "linear")(dict(vocab=301, width=72), dict(weight="h"))
    head.bind(on_gpu(t), rt)
    for rows in (2, 30, 150):   # one skinny product, one with several row tiles, chunks of 64 rows
        x = torch.randn(rows, 72, generator=torch.Generator().manual_seed(7)).to(rt.dtype)
        y = head.forward(x.to("cuda"))
        assert y.dtype == torch.float32 and y.shape == (rows, 301)
        assert rel(y, x.double().numpy() @ tn["h"].T) <= TOL[rt.dtype]


def test_pre_norm_block(rt):
    from burn_lm_amd import registry
    from burn_lm_amd.cache.cache import Cache
    from burn_lm_amd.engine.batch import build_step
    D, heads, kvh, hd, inner = 72, 6, 2, 12, 100
    t, tn = weights(rt, 8, q=(heads * hd, D), k=(kvh * hd, D), v=(kvh * hd, D), o=(D, heads * hd),
                    g=(inner, D), u=(inner, D), d=(D, inner), n1=(D,), n2=(D,))
    rope = registry.part("position", "rope")(dict(head_dim=hd, theta=10000.0, pairing="interleaved", scaling=None), {})
    rope.bind({}, rt); rope.prepare(64, rt)
    parts = [registry.part("mixer", "attention")(dict(width=D, heads=heads, kv_heads=kvh, head_dim=hd,
                                                      scale=1 / math.sqrt(hd), position=rope),
                                                 dict(q="q", k="k", v="v", o="o")),
             registry.part("feed_forward", "swiglu")(dict(width=D, inner=inner), dict(gate="g", up="u", down="d")),
             registry.part("norm", "rmsnorm")(dict(width=D, eps=1e-5), dict(weight="n1")),
             registry.part("norm", "rmsnorm")(dict(width=D, eps=1e-5), dict(weight="n2"))]
    for p in parts:
        p.bind(on_gpu(t), rt)
    block = registry.part("block", "pre_norm")(dict(mixer=parts[0], feed_forward=parts[1], mixer_norm=parts[2], ffn_norm=parts[3]))
    cache = Cache([parts[0].cache_need()], [None], 256, 2, 64, PAGE, rt.dtype, rt.device)
    s = cache.open()
    cache.reserve([(s, 19)])
    step = build_step([(s, [0] * 19, [])], cache, rt.device)
    x0 = torch.randn(19, D, generator=torch.Generator().manual_seed(9))
    pending = (torch.randn(19, D, generator=torch.Generator().manual_seed(10)) * 0.1).to(rt.dtype)
    h = x0.to("cuda")
    delta = block.forward(h, pending.to("cuda"), step, cache.views[0])
    lw = dict(wq=tn["q"], wk=tn["k"], wv=tn["v"], wo=tn["o"], w1=tn["g"], w3=tn["u"], w2=tn["d"],
              attention_norm=tn["n1"], ffn_norm=tn["n2"])
    x_in = (x0 + pending.float()).double().numpy()[None]
    want = P.block(x_in, lw, dict(n_heads=heads, n_kv_heads=kvh, head_dim=hd, eps=1e-5), P.rope_base_frequencies(hd, 1e4))[0]
    got = h.double().cpu().numpy() + delta.double().cpu().numpy()     # the block's last add is still pending
    assert float(np.abs(got - want).max() / np.abs(want).max()) <= TOL[rt.dtype]
